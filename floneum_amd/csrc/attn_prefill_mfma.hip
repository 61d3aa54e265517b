// Prefill attention for f16 / bf16 on the gfx950 matrix cores.
//
// Workgroup = 4 wavefronts = 128 query rows of one (batch, head); each wavefront owns 32 rows.
// Keys/values are walked in tiles of 64 rows staged through LDS.  Per tile and wavefront:
//   S^T (64 keys x 32 queries)  = K_tile . Q^T      v_mfma_f32_32x32x16  (A = K from LDS, B = Q in registers)
//   online softmax down the key axis: with S^T every lane owns ONE query column and 16 keys of
//   it per 32-key block, so the row max / row sum are in-lane folds plus one exchange with the
//   lane 32 away (v_permlane32_swap)
//   O^T (D x 32 queries)       += V_tile^T . P^T    A = V^T read from row-major LDS with the
//   transposing LDS load ds_read_b64_tr_b16, B = P^T taken straight from the S^T accumulator
//   registers (the contraction index is permuted identically on both operands)
// All accumulation is f32; P is rounded to the input type for the second product.
// Masking is analytic (causal with offset, sliding window, per-batch kv length, tail of the key
// axis); key tiles that are invisible to the whole workgroup are never loaded, and tiles fully
// visible to a wavefront skip the per-element test.
//
// Reference semantics: fusor-ml/fusor/src/composite/flash_attention.rs:141-199, f32 accumulation
// of 16-bit inputs as fusor-ml/core/src/composite/flash_attention.rs:186-203,323-327; head
// mapping kv_head = head / (H / Hkv) (core :135-137,163-167).
#include "common.h"
#include "device_utils.h"

namespace fhip {

constexpr int PF_WAVES = 4;
constexpr int PF_BM = 32 * PF_WAVES;  // query rows per workgroup
constexpr int PF_BN = 64;             // key rows per tile
constexpr float PF_LOG2E = 1.4426950408889634f;

#define LDS_PTR(type, byte_off) ((__attribute__((address_space(3))) type *)(lds_base + (byte_off)))

template <typename T>
struct Mma;
template <>
struct Mma<half_t> {
    typedef half8_t vec8;
    static __device__ __forceinline__ float16_t mfma(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float x, float y) {
        half2_t h = {(half_t)x, (half_t)y};
        return __builtin_bit_cast(uint32_t, h);
    }
};
template <>
struct Mma<bf16_t> {
    typedef bf16x8_t vec8;
    static __device__ __forceinline__ float16_t mfma(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float x, float y) {
        return (uint32_t)from_float<bf16_t>(x).bits | ((uint32_t)from_float<bf16_t>(y).bits << 16);
    }
};

template <int D>
struct PfCfg {
    static constexpr int KP = D * 2 + 16;                            // K tile row pitch, bytes
    static constexpr int VP = (D == 64) ? 192 : 320;                 // V tile row pitch, bytes
    static constexpr int K_BYTES = PF_BN * KP;
    static constexpr int V_BYTES = PF_BN * VP;
    static constexpr int CPR = D / 8;                                // 16-byte chunks per row
    static constexpr int NCH = PF_BN * CPR / (64 * PF_WAVES);        // chunks per thread per tile
};

__device__ __forceinline__ float half_swap_max(float x) {
    // max of x with the value held by the lane 32 away
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <typename T, int D>
__global__ __launch_bounds__(64 * PF_WAVES, 2) void prefill_mfma_kernel(AttnParams p, int nqb) {
    typedef PfCfg<D> C;
    typedef typename Mma<T>::vec8 vec8;
    __shared__ __attribute__((aligned(16))) char smem[C::K_BYTES + C::V_BYTES];
    auto lds_base = (__attribute__((address_space(3))) char *)smem;

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int ln = lane & 31;  // query column / key row owned inside a 32-wide MFMA block
    const int h2 = lane >> 5;  // which half of the contraction slice

    // workgroup -> (query block, batch, head): long query blocks first, and heads laid out so
    // the workgroups that land on one XCD (id % 8) share a KV head whenever H is a multiple of 8
    const int bh_count = p.B * p.H;
    const int id = blockIdx.x;
    const int qb = nqb - 1 - id / bh_count;
    int rem = id % bh_count;
    const int b = rem / p.H;
    int h = rem % p.H;
    if ((p.H & 7) == 0) h = (h & 7) * (p.H >> 3) + (h >> 3);
    const int g = h / p.G;

    const int q0 = qb * PF_BM;
    const int qw0 = q0 + 32 * wave;
    const int query = qw0 + ln;
    const int off = (int)p.q_pos_offset;

    int kv_hi = p.Skv;
    if (p.kv_lens) kv_hi = min(kv_hi, max(p.kv_lens[b], 0));

    // key range visible to the workgroup / to this wavefront
    const int q_last_wg = min(q0 + PF_BM - 1, p.Sq - 1);
    const int q_last_w = min(qw0 + 31, p.Sq - 1);
    int hi_wg = kv_hi, lo_wg = 0, hi_w = kv_hi, lo_w = 0;
    if (p.analytic) {
        if (p.causal) {
            hi_wg = (int)min((int64_t)kv_hi, (int64_t)q_last_wg + off + 1);
            hi_w = (int)min((int64_t)kv_hi, (int64_t)q_last_w + off + 1);
        }
        if (p.window > 0) {
            lo_wg = (int)max((int64_t)0, (int64_t)q0 + off - p.window + 1);
            lo_w = (int)max((int64_t)0, (int64_t)qw0 + off - p.window + 1);
        }
    }
    const bool wave_has_rows = qw0 < p.Sq;

    // Q^T operand: Q[query][16 kb + 8 h2 .. +8], kept in registers for the whole kernel
    vec8 qreg[D / 16];
    {
        const int qrow = min(query, p.Sq - 1);
        const uint16_t *qp = (const uint16_t *)p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)qrow * p.qs[2];
#pragma unroll
        for (int kb = 0; kb < D / 16; kb++) {
            uint4_t raw = *(const uint4_t *)(qp + 16 * kb + 8 * h2);
            qreg[kb] = __builtin_bit_cast(vec8, raw);
        }
    }

    const uint16_t *kg = (const uint16_t *)p.k + b * p.ks[0] + g * p.ks[1];
    const uint16_t *vg = (const uint16_t *)p.v + b * p.vs[0] + g * p.vs[1];

    float16_t o[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    const float scale2 = p.scale * PF_LOG2E;

    uint4_t kst[C::NCH], vst[C::NCH];
    auto load_tile = [&](int j0) {
#pragma unroll
        for (int i = 0; i < C::NCH; i++) {
            const int cid = tid + 64 * PF_WAVES * i;
            const int row = cid / C::CPR, col = cid % C::CPR;
            const int key = min(j0 + row, p.Skv - 1);
            kst[i] = *(const uint4_t *)(kg + (int64_t)key * p.ks[2] + col * 8);
            vst[i] = *(const uint4_t *)(vg + (int64_t)key * p.vs[2] + col * 8);
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < C::NCH; i++) {
            const int cid = tid + 64 * PF_WAVES * i;
            const int row = cid / C::CPR, col = cid % C::CPR;
            *LDS_PTR(uint4_t, row * C::KP + col * 16) = kst[i];
            *LDS_PTR(uint4_t, C::K_BYTES + row * C::VP + col * 16) = vst[i];
        }
    };

    const int j_begin = (lo_wg / PF_BN) * PF_BN;
    if (j_begin < hi_wg) load_tile(j_begin);

    for (int j0 = j_begin; j0 < hi_wg; j0 += PF_BN) {
        __syncthreads();  // everyone finished reading the previous tile
        store_tile();
        __syncthreads();
        if (j0 + PF_BN < hi_wg) load_tile(j0 + PF_BN);

        const bool tile_visible = wave_has_rows && j0 < hi_w && j0 + PF_BN > lo_w;
        if (!tile_visible) continue;

        // ---- S^T = K . Q^T --------------------------------------------------------------------
        float16_t s[2];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) s[t][r] = 0.0f;
#pragma unroll
        for (int kb = 0; kb < D / 16; kb++) {
#pragma unroll
            for (int t = 0; t < 2; t++) {
                uint4_t raw = *LDS_PTR(uint4_t, (32 * t + ln) * C::KP + kb * 32 + h2 * 16);
                s[t] = Mma<T>::mfma(__builtin_bit_cast(vec8, raw), qreg[kb], s[t]);
            }
        }

        // ---- mask ------------------------------------------------------------------------------
        // element r of block t is key j0 + 32 t + 8 (r / 4) + 4 h2 + r % 4 for query `query`
        bool full = j0 + PF_BN <= kv_hi;
        if (p.analytic) {
            if (p.causal) full = full && (j0 + PF_BN - 1 <= qw0 + off);
            if (p.window > 0) full = full && ((int64_t)j0 + p.window > (int64_t)q_last_w + off);
        }
        if (!full) {
            const int qpos = query + off;
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int key = j0 + 32 * t + 8 * (r >> 2) + 4 * h2 + (r & 3);
                    bool vis = key < kv_hi;
                    if (p.analytic) {
                        if (p.causal) vis = vis && key <= qpos;
                        if (p.window > 0) vis = vis && ((int64_t)key + p.window > (int64_t)qpos);
                    }
                    s[t][r] = vis ? s[t][r] : -INFINITY;
                }
        }

        // ---- online softmax (log2 domain) ------------------------------------------------------
        float mx = s[0][0];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[t][r]);
        mx = half_swap_max(mx);
        const float m_new = fmaxf(m, mx * scale2);
        const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
        const float corr = __builtin_amdgcn_exp2f(m - m_safe);
        m = m_new;
        float psum = 0.0f;
        uint32_t pk[2][8];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                const float p0 = __builtin_amdgcn_exp2f(fmaf(s[t][r], scale2, -m_safe));
                const float p1 = __builtin_amdgcn_exp2f(fmaf(s[t][r + 1], scale2, -m_safe));
                psum += p0 + p1;
                pk[t][r >> 1] = Mma<T>::pack2(p0, p1);
            }
        l = l * corr + psum;
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[db][r] *= corr;

        // ---- O^T += V^T . P^T ------------------------------------------------------------------
        // contraction slice (t, kk): this half-wave's keys are 32 t + 16 kk + 4 h2 + {0..3} and + 8
        const int i16 = lane & 15;
        const int bl = (lane & 31) >> 4;
#pragma unroll
        for (int t = 0; t < 2; t++) {
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
                uint4_t braw = {pk[t][4 * kk], pk[t][4 * kk + 1], pk[t][4 * kk + 2], pk[t][4 * kk + 3]};
                const vec8 bop = __builtin_bit_cast(vec8, braw);
                const int krow = 32 * t + 16 * kk + 4 * h2 + (i16 >> 2);
#pragma unroll
                for (int db = 0; db < D / 32; db++) {
                    const int colb = (32 * db + 16 * bl + 4 * (i16 & 3)) * 2;
                    short4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        LDS_PTR(short4_t, C::K_BYTES + krow * C::VP + colb));
                    short4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        LDS_PTR(short4_t, C::K_BYTES + (krow + 8) * C::VP + colb));
                    uint4_t araw = {__builtin_bit_cast(uint2_t, a0)[0], __builtin_bit_cast(uint2_t, a0)[1],
                                    __builtin_bit_cast(uint2_t, a1)[0], __builtin_bit_cast(uint2_t, a1)[1]};
                    o[db] = Mma<T>::mfma(__builtin_bit_cast(vec8, araw), bop, o[db]);
                }
            }
        }
    }

    // ---- epilogue: out[query][dim] = O^T[dim][query] / l ----------------------------------------
    const float l_tot = half_swap_sum(l);
    if (query < p.Sq) {
        const float inv = 1.0f / l_tot;  // no visible key: l = 0 -> 0 * inf = NaN, like the reference
        const int64_t obase = b * p.os[0] + h * p.os[1] + (int64_t)query * p.os[2];
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int dim = 32 * db + 8 * (r >> 2) + 4 * h2 + (r & 3);
                const float val = (l_tot == 0.0f) ? __builtin_nanf("") : o[db][r] * inv;
                if (p.out_f32) ((float *)p.out)[obase + dim * p.os[3]] = val;
                else ((T *)p.out)[obase + dim * p.os[3]] = from_float<T>(val);
            }
    }
}

template <typename T>
static int launch_t(const AttnParams &p, hipStream_t stream) {
    const int nqb = (p.Sq + PF_BM - 1) / PF_BM;
    const long blocks = (long)nqb * p.B * p.H;
    if (blocks > 0x7fffffffL) {
        set_error("prefill: too many workgroups (%ld)", blocks);
        return FHIP_ERR_UNSUPPORTED;
    }
    dim3 grid((unsigned)blocks), block(64 * PF_WAVES);
    switch (p.D) {
        case 64: hipLaunchKernelGGL((prefill_mfma_kernel<T, 64>), grid, block, 0, stream, p, nqb); break;
        case 96: hipLaunchKernelGGL((prefill_mfma_kernel<T, 96>), grid, block, 0, stream, p, nqb); break;
        case 128: hipLaunchKernelGGL((prefill_mfma_kernel<T, 128>), grid, block, 0, stream, p, nqb); break;
        default: set_error("prefill MFMA kernel: head_dim %d not in {64, 96, 128}", p.D); return FHIP_ERR_UNSUPPORTED;
    }
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

int launch_prefill_mfma(const AttnParams &p, fhip_dtype dtype, hipStream_t stream) {
    if (dtype == FHIP_F16) return launch_t<half_t>(p, stream);
    if (dtype == FHIP_BF16) return launch_t<bf16_t>(p, stream);
    set_error("prefill MFMA kernel takes f16/bf16 only");
    return FHIP_ERR_UNSUPPORTED;
}

}  // namespace fhip
