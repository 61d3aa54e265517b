// Dense additive masks as intervals.
//
// fusor hands the attention operator its masks as tensors (fusor-ml/fusor/src/cache/mask_cache.rs:36-116,
// attention_mask.rs:26-46): 0 where a key is visible, -inf where it is not.  Every mask those builders
// produce (causal, sliding window, their concatenation with a cached prefix) and every padding mask
// has, per row, ONE run of zeros.  This kernel checks that per row and writes the run as {lo, hi}; the
// tiled attention kernels then mask by interval and never read the [rows, kv_seq_len] tensor again.  A
// row that is anything else (finite biases, several runs, NaN) marks *bad with the call's tag and the call falls
// back to a kernel that adds the mask values as the reference does
// (fusor-ml/fusor/src/composite/flash_attention.rs:161-176).
//
// The other direction lives here too: mask_build_kernel writes the tensor MaskCache::get_mask would build
// (mask_cache.rs:36-116) straight into device memory, for callers that want the tensor without the O(seq^2)
// host loop and the upload.
#include "common.h"
#include "device_utils.h"

namespace fhip {

constexpr int MI_WAVES = 4;

// EB: element bytes; NINF16: the 16-bit pattern of -inf (0xFC00 f16, 0xFF80 bf16), unused for EB == 4
template <int EB>
__global__ __launch_bounds__(64 * MI_WAVES) void mask_intervals_kernel(const char *mask, int64_t ms0, int64_t ms1,
                                                                      int rows, int cols, uint32_t ninf16, int vec_ok,
                                                                      int2 *iv, int32_t *bad, int32_t bad_tag) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * MI_WAVES + (threadIdx.x >> 6);
    if (row >= rows) return;  // whole wavefront
    const char *mrow = mask + (int64_t)row * ms0 * EB;
    int lo = 0x7fffffff, hi = 0, zeros = 0, others = 0;
    auto take = [&](int j, uint32_t bits) {
        bool ninf, zero;
        if (EB == 4) {
            ninf = bits == 0xFF800000u;
            zero = (bits & 0x7FFFFFFFu) == 0;
        } else {
            ninf = bits == ninf16;
            zero = (bits & 0x7FFFu) == 0;
        }
        if (!ninf) {
            lo = min(lo, j);
            hi = max(hi, j + 1);
            zeros += zero ? 1 : 0;
            others += zero ? 0 : 1;
        }
    };
    if (vec_ok) {
        // contiguous, 16-byte aligned rows: 16 bytes per lane and step
        constexpr int EPV = 16 / EB;
        const int nvec = cols / EPV;
        // a piece that is all -inf or all zero (nearly every piece of a real mask) is settled with four word
        // compares; four pieces are in flight per lane
        const uint32_t ninf_word = EB == 4 ? 0xFF800000u : (ninf16 | (ninf16 << 16));
        const uint32_t abs_word = EB == 4 ? 0x7FFFFFFFu : 0x7FFF7FFFu;
        auto take_piece = [&](int c, const uint4_t raw) {
            const bool all_ninf = raw[0] == ninf_word && raw[1] == ninf_word && raw[2] == ninf_word && raw[3] == ninf_word;
            if (all_ninf) return;
            if (((raw[0] | raw[1] | raw[2] | raw[3]) & abs_word) == 0) {
                lo = min(lo, c * EPV);
                hi = max(hi, c * EPV + EPV);
                zeros += EPV;
                return;
            }
#pragma unroll
            for (int e = 0; e < EPV; e++) {
                uint32_t bits;
                if (EB == 4) bits = raw[e];
                else bits = (raw[e >> 1] >> (16 * (e & 1))) & 0xffffu;
                take(c * EPV + e, bits);
            }
        };
        int c = lane;
        for (; c + 192 < nvec; c += 256) {
            uint4_t raw[4];
#pragma unroll
            for (int u = 0; u < 4; u++) raw[u] = __builtin_nontemporal_load((const uint4_t *)(mrow) + c + 64 * u);
#pragma unroll
            for (int u = 0; u < 4; u++) take_piece(c + 64 * u, raw[u]);
        }
        for (; c < nvec; c += 64) take_piece(c, __builtin_nontemporal_load((const uint4_t *)(mrow) + c));
        for (int j = nvec * EPV + lane; j < cols; j += 64) {
            uint32_t bits = EB == 4 ? *(const uint32_t *)(mrow + (int64_t)j * 4) : *(const uint16_t *)(mrow + (int64_t)j * 2);
            take(j, bits);
        }
    } else {
        for (int j = lane; j < cols; j += 64) {
            const char *e = mrow + (int64_t)j * ms1 * EB;
            uint32_t bits = EB == 4 ? *(const uint32_t *)e : *(const uint16_t *)e;
            take(j, bits);
        }
    }
    lo = wave_reduce_i(lo, [](int a, int b) { return min(a, b); });
    hi = wave_reduce_i(hi, [](int a, int b) { return max(a, b); });
    zeros = wave_reduce_i(zeros, [](int a, int b) { return a + b; });
    others = __builtin_amdgcn_ballot_w64(others != 0) != 0 ? 1 : 0;
    if (lane == 0) {
        if (hi == 0) lo = 0;  // no visible key at all: the empty interval
        const bool ok = others == 0 && zeros == hi - lo;  // only zeros and -inf, and the zeros are one run
        iv[row] = int2{lo, hi};
        if (!ok) *(volatile int32_t *)bad = bad_tag;  // every such row stores the same value
    }
}

size_t mask_intervals_bytes(int rows) { return ((size_t)rows * sizeof(int2) + 16 + 15) & ~(size_t)15; }

int launch_mask_intervals(const AttnParams &p, fhip_dtype dtype, int2 *iv, int32_t *bad, hipStream_t stream) {
    const int rows = p.mask_kind == FHIP_MASK_QK ? p.Sq : p.B;
    const int cols = p.Skv;
    if (rows == 0) return FHIP_OK;
    const int eb = dtype == FHIP_F32 ? 4 : 2;
    const int vec_ok = (p.ms1 == 1 || cols <= 1) && ((uintptr_t)p.mask % 16 == 0) && ((p.ms0 * eb) % 16 == 0);
    dim3 grid((rows + MI_WAVES - 1) / MI_WAVES), block(64 * MI_WAVES);
    if (eb == 4)
        hipLaunchKernelGGL(mask_intervals_kernel<4>, grid, block, 0, stream, (const char *)p.mask, p.ms0, p.ms1, rows, cols,
                           0u, vec_ok, iv, bad, p.bad_tag);
    else
        hipLaunchKernelGGL(mask_intervals_kernel<2>, grid, block, 0, stream, (const char *)p.mask, p.ms0, p.ms1, rows, cols,
                           dtype == FHIP_F16 ? 0xFC00u : 0xFF80u, vec_ok, iv, bad, p.bad_tag);
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

// element (i, j) of get_mask(seq_len, seqlen_offset, window): columns below `off` are visible cached keys, the
// rest is the causal (j - off > i) or sliding-window (i < j - off or j - off + window <= i) base mask
template <typename W>
__global__ __launch_bounds__(256) void mask_build_kernel(W *out, uint32_t rows, uint64_t cols, uint64_t off, int has_window,
                                                         uint64_t window, W ninf) {
    const uint64_t total = (uint64_t)rows * cols;
    for (uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (uint64_t)gridDim.x * 256) {
        const uint64_t i = idx / cols, c = idx % cols;
        bool masked = false;
        if (c >= off) {
            const uint64_t j = c - off;
            masked = has_window ? (i < j || j + window <= i) : (j > i);
        }
        out[idx] = masked ? ninf : (W)0;
    }
}

// the same, 16 bytes per lane and step (V = 4 f32 or 8 16-bit elements of one row; cols % V == 0, out 16-byte aligned)
template <typename W, int V>
__global__ __launch_bounds__(256) void mask_build_wide_kernel(W *out, uint32_t rows, uint64_t cols, uint64_t off, int has_window,
                                                              uint64_t window, W ninf) {
    const uint64_t per_row = cols / V, total = (uint64_t)rows * per_row;
    for (uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (uint64_t)gridDim.x * 256) {
        const uint64_t i = idx / per_row, c0 = (idx % per_row) * V;
        W vals[V];
#pragma unroll
        for (int e = 0; e < V; e++) {
            const uint64_t c = c0 + e;
            bool masked = false;
            if (c >= off) {
                const uint64_t j = c - off;
                masked = has_window ? (i < j || j + window <= i) : (j > i);
            }
            vals[e] = masked ? ninf : (W)0;
        }
        uint4_t raw;
        __builtin_memcpy(&raw, vals, 16);
        *(uint4_t *)(out + i * cols + c0) = raw;
    }
}

int launch_mask_build(void *out, fhip_dtype dtype, uint32_t rows, uint64_t cols, uint64_t off, int has_window,
                      uint64_t window, hipStream_t stream) {
    const uint64_t total = (uint64_t)rows * cols;
    if (total == 0) return FHIP_OK;
    const int V = dtype == FHIP_F32 ? 4 : 8;
    const bool wide = cols % V == 0 && ((uintptr_t)out % 16) == 0;
    const uint64_t blocks = ((wide ? total / V : total) + 255) / 256;
    const dim3 grid((unsigned)(blocks < 65536 * 4 ? blocks : 65536 * 4)), block(256);
    if (dtype == FHIP_F32) {
        if (wide)
            hipLaunchKernelGGL((mask_build_wide_kernel<uint32_t, 4>), grid, block, 0, stream, (uint32_t *)out, rows, cols, off,
                               has_window, window, 0xFF800000u);
        else
            hipLaunchKernelGGL(mask_build_kernel<uint32_t>, grid, block, 0, stream, (uint32_t *)out, rows, cols, off, has_window,
                               window, 0xFF800000u);
    } else {
        const uint16_t ninf = (uint16_t)(dtype == FHIP_F16 ? 0xFC00u : 0xFF80u);
        if (wide)
            hipLaunchKernelGGL((mask_build_wide_kernel<uint16_t, 8>), grid, block, 0, stream, (uint16_t *)out, rows, cols, off,
                               has_window, window, ninf);
        else
            hipLaunchKernelGGL(mask_build_kernel<uint16_t>, grid, block, 0, stream, (uint16_t *)out, rows, cols, off, has_window,
                               window, ninf);
    }
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

}  // namespace fhip
