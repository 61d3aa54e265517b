// Prefill attention for f32 tensors on the gfx950 f32 matrix instruction (v_mfma_f32_32x32x2_f32).
//
// Same decomposition as the 16-bit kernel: a workgroup of 4 wavefronts owns 128 query rows of one
// (batch, head), a wavefront 32 of them; K/V tiles of 32 rows pass through LDS.
//   S^T (32 keys x 32 queries) = K_tile . Q^T   A = K[key][dim] from LDS (128-bit reads, the four
//                                               values feed four MFMA steps), B = Q in registers
//   softmax down the key axis: every lane owns one query and 16 keys -> in-lane folds plus one
//   exchange with the lane 32 away
//   O^T (D x 32 queries) += V^T . P^T           A = V[key][dim] read row-major (one f32 per lane),
//                                               B = the S^T accumulator registers themselves
// Products and sums are f32 throughout (no reduced-precision operand), which is what the f32
// tolerance (relative L2 1e-5 against the reference's f32 CPU path) needs.
//
// Reference semantics: fusor-ml/fusor/src/composite/flash_attention.rs:141-199; this is the data
// type kalosm-llama always calls with (models/kalosm-llama/src/raw/attention_layer.rs:400-448).
#include "attn_bounds.h"
#include "common.h"
#include "device_utils.h"

namespace fhip {

constexpr int PF32_WAVES = 4;
constexpr int PF32_BM = 32 * PF32_WAVES;
constexpr int PF32_BN = 32;
constexpr float PF32_LOG2E = 1.4426950408889634f;

#define LDS32_PTR(type, byte_off) ((__attribute__((address_space(3))) type *)(lds_base + (byte_off)))

__device__ __forceinline__ float half_swap_max32(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum32(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <int D>
__global__ __launch_bounds__(64 * PF32_WAVES, 2) void prefill_f32_kernel(AttnParams p, int nqb) {
    constexpr int KP = D * 4 + 16;  // row pitch in bytes: rows 4 banks apart -> conflict-free b128 reads
    constexpr int K_BYTES = PF32_BN * KP;
    constexpr int CPR = D / 4;      // 16-byte chunks per row
    constexpr int NCH = PF32_BN * CPR / (64 * PF32_WAVES);
    __shared__ __attribute__((aligned(16))) char smem[2 * K_BYTES];
    auto lds_base = (__attribute__((address_space(3))) char *)smem;

    if (p.iv_bad && *p.iv_bad != 0) return;  // the mask is not made of intervals: the general kernel takes the call
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int ln = lane & 31;
    const int h2 = lane >> 5;

    const int bh_count = p.B * p.H;
    const int id = blockIdx.x;
    const int qb = nqb - 1 - id / bh_count;
    int rem = id % bh_count;
    const int b = rem / p.H;
    int h = rem % p.H;
    if ((p.H & 7) == 0) h = (h & 7) * (p.H >> 3) + (h >> 3);
    const int g = h / p.G;

    const int q0 = qb * PF32_BM;
    const int qw0 = q0 + 32 * wave;
    const int query = qw0 + ln;
    const RowBounds rb = row_bounds(p, b, q0, PF32_BM, qw0, lane);
    const int lo_wg = rb.lo_wg, hi_wg = rb.hi_wg, lo_w = rb.lo_w, hi_w = rb.hi_w;
    const bool wave_has_rows = qw0 < p.Sq;

    // Q operand: Q[query][8 kc + 4 h2 .. +4]
    float4_t qreg[D / 8];
    {
        const int qrow = min(query, p.Sq - 1);
        const float *qp = (const float *)p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)qrow * p.qs[2];
#pragma unroll
        for (int kc = 0; kc < D / 8; kc++) qreg[kc] = *(const float4_t *)(qp + 8 * kc + 4 * h2);
    }
    const float *kg = (const float *)p.k + b * p.ks[0] + g * p.ks[1];
    const float *vg = (const float *)p.v + b * p.vs[0] + g * p.vs[1];

    float16_t o[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    const float scale2 = p.scale * PF32_LOG2E;

    float4_t kst[NCH], vst[NCH];
    auto load_tile = [&](int j0) {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int cid = tid + 64 * PF32_WAVES * i;
            const int row = cid / CPR, col = cid % CPR;
            const int key = min(j0 + row, p.Skv - 1);
            kst[i] = *(const float4_t *)(kg + (int64_t)key * p.ks[2] + col * 4);
            vst[i] = *(const float4_t *)(vg + (int64_t)key * p.vs[2] + col * 4);
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int cid = tid + 64 * PF32_WAVES * i;
            const int row = cid / CPR, col = cid % CPR;
            *LDS32_PTR(float4_t, row * KP + col * 16) = kst[i];
            *LDS32_PTR(float4_t, K_BYTES + row * KP + col * 16) = vst[i];
        }
    };

    const int j_begin = (lo_wg / PF32_BN) * PF32_BN;
    if (j_begin < hi_wg) load_tile(j_begin);

    for (int j0 = j_begin; j0 < hi_wg; j0 += PF32_BN) {
        lds_barrier();  // everyone finished reading the previous tile (LDS-only barrier: the prefetch
        store_tile();   // issued below stays in flight across the math)
        lds_barrier();
        if (j0 + PF32_BN < hi_wg) load_tile(j0 + PF32_BN);

        const bool tile_visible = wave_has_rows && j0 < hi_w && j0 + PF32_BN > lo_w;
        if (!tile_visible) continue;

        // S^T: contraction step (kc, i) uses dim 8 kc + 4 h2 + i on both operands
        float16_t s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.0f;
#pragma unroll
        for (int kc = 0; kc < D / 8; kc++) {
            const float4_t a = *LDS32_PTR(float4_t, ln * KP + (8 * kc + 4 * h2) * 4);
#pragma unroll
            for (int i = 0; i < 4; i++) s = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], qreg[kc][i], s, 0, 0, 0);
        }

        // element r is key j0 + 8 (r / 4) + 4 h2 + r % 4 for query `query`
        if (!(j0 >= rb.full_lo_w && j0 + PF32_BN <= rb.full_hi_w)) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int key = j0 + 8 * (r >> 2) + 4 * h2 + (r & 3);
                s[r] = (key >= rb.klo && key < rb.khi) ? s[r] : -INFINITY;
            }
        }

        float mx = s[0];
#pragma unroll
        for (int r = 1; r < 16; r++) mx = fmaxf(mx, s[r]);
        mx = half_swap_max32(mx);
        const float m_new = fmaxf(m, mx * scale2);
        const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
        const float corr = __builtin_amdgcn_exp2f(m - m_safe);
        m = m_new;
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            s[r] = __builtin_amdgcn_exp2f(fmaf(s[r], scale2, -m_safe));
            psum += s[r];
        }
        l = l * corr + psum;
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[db][r] *= corr;

        // O^T += V^T . P^T: contraction step r pairs this half-wave's key 8 (r/4) + 4 h2 + r%4
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int krow = 8 * (r >> 2) + 4 * h2 + (r & 3);
#pragma unroll
            for (int db = 0; db < D / 32; db++) {
                const float a = *LDS32_PTR(float, K_BYTES + krow * KP + (32 * db + ln) * 4);
                o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, s[r], o[db], 0, 0, 0);
            }
        }
    }

    const float l_tot = half_swap_sum32(l);
    if (query < p.Sq) {
        float *op = (float *)p.out + b * p.os[0] + h * p.os[1] + (int64_t)query * p.os[2];
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int dim = 32 * db + 8 * (r >> 2) + 4 * h2 + (r & 3);
                op[dim * p.os[3]] = o[db][r] / l_tot;  // no visible key: 0/0 = NaN like the reference
            }
    }
}

int launch_prefill_f32(const AttnParams &p, hipStream_t stream) {
    const int nqb = (p.Sq + PF32_BM - 1) / PF32_BM;
    const long blocks = (long)nqb * p.B * p.H;
    if (blocks > 0x7fffffffL) {
        set_error("prefill f32: too many workgroups (%ld)", blocks);
        return FHIP_ERR_UNSUPPORTED;
    }
    dim3 grid((unsigned)blocks), block(64 * PF32_WAVES);
    switch (p.D) {
        case 32: hipLaunchKernelGGL(prefill_f32_kernel<32>, grid, block, 0, stream, p, nqb); break;
        case 64: hipLaunchKernelGGL(prefill_f32_kernel<64>, grid, block, 0, stream, p, nqb); break;
        case 96: hipLaunchKernelGGL(prefill_f32_kernel<96>, grid, block, 0, stream, p, nqb); break;
        case 128: hipLaunchKernelGGL(prefill_f32_kernel<128>, grid, block, 0, stream, p, nqb); break;
        default: set_error("prefill f32 kernel: head_dim %d not in {32, 64, 96, 128}", p.D); return FHIP_ERR_UNSUPPORTED;
    }
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

}  // namespace fhip
