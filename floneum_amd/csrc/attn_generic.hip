// Generic attention kernel: any element type, any strides, any additive mask, head_dim <= 512.
// One wavefront owns one query row (b, h, i); four rows per 256-thread workgroup.  Lanes split the
// keys of a 64-key tile for QK^T, then split head_dim for PV; the probabilities of the tile are
// broadcast lane by lane.  Accumulation is f32 throughout and the softmax is the online form of
//   s = (q.k) * scale + mask;  p = exp(s - max s);  out = sum_j p_j v_j / sum_j p_j
// (reference semantics: fusor-ml/fusor/src/composite/flash_attention.rs:141-199).
// It is the fallback for shapes the tiled kernels do not take and the on-device cross-check.
#include "common.h"
#include "device_utils.h"

namespace fhip {

constexpr int GEN_WAVES = 4;
constexpr int GEN_MAXT = 8;  // head_dim <= 64 * GEN_MAXT

template <typename T>
__global__ __launch_bounds__(64 * GEN_WAVES) void attn_generic_kernel(AttnParams p) {
    __shared__ float q_lds[GEN_WAVES][512];
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * GEN_WAVES + wave;
    const int64_t total = (int64_t)p.B * p.H * p.Sq;
    if (row >= total) return;  // whole wavefront leaves together; no workgroup barrier is used below
    if (p.only_if_bad && *p.only_if_bad != p.bad_tag) return;  // a tiled kernel has taken this call
    const int i = (int)(row % p.Sq);
    const int h = (int)((row / p.Sq) % p.H);
    const int b = (int)(row / ((int64_t)p.Sq * p.H));
    const int g = h / p.G;  // GQA head mapping (reference: flash_attention.rs:101-138)

    const T *q = (const T *)p.q + b * p.qs[0] + h * p.qs[1] + i * p.qs[2];
    const T *kbase = (const T *)p.k + b * p.ks[0] + g * p.ks[1];
    const T *vbase = (const T *)p.v + b * p.vs[0] + g * p.vs[1];
    const int D = p.D;
    for (int d = lane; d < D; d += 64) q_lds[wave][d] = to_float(q[d * p.qs[3]]);
    wave_lds_sync();

    int kv_hi = p.Skv;
    if (p.kv_lens) {
        int len = p.kv_lens[b];
        kv_hi = len < kv_hi ? (len < 0 ? 0 : len) : kv_hi;
    }
    const T *mrow = nullptr;
    if (p.mask_kind == FHIP_MASK_QK) mrow = (const T *)p.mask + i * p.ms0;
    if (p.mask_kind == FHIP_MASK_BATCH_KEY) mrow = (const T *)p.mask + b * p.ms0;

    float m = -INFINITY, l = 0.0f;
    float acc[GEN_MAXT];
#pragma unroll
    for (int t = 0; t < GEN_MAXT; t++) acc[t] = 0.0f;

    for (int j0 = 0; j0 < kv_hi; j0 += 64) {
        const int j = j0 + lane;
        float s = -INFINITY;
        if (j < kv_hi) {
            const T *kr = kbase + j * p.ks[2];
            float dot = 0.0f;
            for (int d = 0; d < D; d++) dot = fmaf(q_lds[wave][d], to_float(kr[d * p.ks[3]]), dot);
            s = dot * p.scale;
            if (mrow) s = s + to_float(mrow[j * p.ms1]);
            if (p.analytic) {
                const int64_t qpos = (int64_t)i + p.q_pos_offset;
                if (p.causal && (int64_t)j > qpos) s = -INFINITY;
                if (p.window > 0 && (int64_t)j + p.window <= qpos) s = -INFINITY;
            }
        }
        const float tile_max = wave_max(s);
        const float m_new = fmaxf(m, tile_max);
        if (m_new == -INFINITY) continue;  // nothing visible yet (uniform across the wavefront)
        const float pj = expf(s - m_new);  // s = -inf -> 0
        const float corr = expf(m - m_new);  // m = -inf -> 0
        l = l * corr + wave_sum(pj);
        m = m_new;
        const int nj = (kv_hi - j0) < 64 ? (kv_hi - j0) : 64;
#pragma unroll
        for (int t = 0; t < GEN_MAXT; t++) {
            const int d = lane + 64 * t;
            if (d < D) {
                float a = acc[t] * corr;
                const T *vc = vbase + (int64_t)j0 * p.vs[2] + d * p.vs[3];
                for (int jj = 0; jj < nj; jj++) a = fmaf(read_lane(pj, jj), to_float(vc[jj * p.vs[2]]), a);
                acc[t] = a;
            }
        }
    }
    // a row with no visible key gives 0/0 = NaN, as the reference does
    char *obase = (char *)p.out;
    const int64_t ooff = b * p.os[0] + h * p.os[1] + i * p.os[2];
#pragma unroll
    for (int t = 0; t < GEN_MAXT; t++) {
        const int d = lane + 64 * t;
        if (d < D) {
            const float o = acc[t] / l;
            const int64_t idx = ooff + d * p.os[3];
            if (p.out_f32 || sizeof(T) == 4)
                ((float *)obase)[idx] = o;
            else
                ((T *)obase)[idx] = from_float<T>(o);
        }
    }
}

int launch_generic(const AttnParams &p, fhip_dtype dtype, hipStream_t stream) {
    if (p.D > 64 * GEN_MAXT) {
        set_error("generic kernel: head_dim %d > %d", p.D, 64 * GEN_MAXT);
        return FHIP_ERR_UNSUPPORTED;
    }
    const int64_t rows = (int64_t)p.B * p.H * p.Sq;
    const int64_t blocks = (rows + GEN_WAVES - 1) / GEN_WAVES;
    if (blocks > 0x7fffffffLL) {
        set_error("generic kernel: too many query rows (%lld)", (long long)rows);
        return FHIP_ERR_UNSUPPORTED;
    }
    dim3 grid((unsigned)blocks), block(64 * GEN_WAVES);
    switch (dtype) {
        case FHIP_F32: FHIP_LAUNCH_MAIN(attn_generic_kernel<float>, grid, block, stream, p, p); break;
        case FHIP_F16: FHIP_LAUNCH_MAIN(attn_generic_kernel<half_t>, grid, block, stream, p, p); break;
        case FHIP_BF16: FHIP_LAUNCH_MAIN(attn_generic_kernel<bf16_t>, grid, block, stream, p, p); break;
    }
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

}  // namespace fhip
