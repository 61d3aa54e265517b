// Split-KV decode attention for a 16-bit KV cache (query length 1).
//
// Pass 1 (decode_splitkv_kernel): grid = (split, batch * kv_head * head_block).  A workgroup of
// four wavefronts streams one chunk of keys/values of one KV head exactly once for all the query
// heads that share it (GQA group), with 128-bit loads laid out so that one wavefront load
// instruction covers 64/LPK whole key rows back to back (LPK lanes x 8 elements per row).
// Every group of LPK lanes keeps its own online-softmax state (m, l, acc) in the log2 domain, so
// the streaming loop needs no cross-lane traffic beyond the LPK-lane dot-product reduction.
// At the end the states are merged (lanes -> wavefront -> workgroup) and written as one partial
// (acc[D], m, l) per (batch, head, split).
// Pass 2 (decode_combine_kernel): log-sum-exp merge of the partials of each (batch, head).
// With a single split pass 1 writes the final output and pass 2 is not launched.
//
// Reference semantics: fusor-ml/fusor/src/composite/flash_attention.rs:141-199 (f32 accumulation
// of 16-bit inputs as in fusor-ml/core/src/composite/flash_attention.rs:186-203,323-327).
#include <cstdlib>

#include "common.h"
#include "device_utils.h"

namespace fhip {

constexpr int DEC_WAVES = 4;
constexpr int DEC_UNROLL = 4;
constexpr float LOG2E = 1.4426950408889634f;

static int env_int(const char *name, int dflt) {
    const char *s = getenv(name);
    if (!s || !*s) return dflt;
    int v = atoi(s);
    return v > 0 ? v : dflt;
}

static int decode_gt(int G) { return G <= 1 ? 1 : G <= 2 ? 2 : G <= 4 ? 4 : 8; }

void decode_plan(int B, int Hkv, int G, int Skv, int D, int compute_units, int *chunk, int *nsplit) {
    (void)D;
    const int gt = decode_gt(G);
    const int hb = (G + gt - 1) / gt;
    const long units = (long)B * Hkv * hb;
    const int wgs_per_cu = env_int("FHIP_DECODE_WGS_PER_CU", 4);
    const int max_chunk = env_int("FHIP_DECODE_MAX_CHUNK", 1024);
    const int min_chunk = env_int("FHIP_DECODE_MIN_CHUNK", 256);
    const long target = (long)compute_units * wgs_per_cu;
    long ns = (target + units - 1) / units;
    const long ns_max = (Skv + min_chunk - 1) / min_chunk;
    const long ns_min = (Skv + max_chunk - 1) / max_chunk;
    if (ns > ns_max) ns = ns_max;
    if (ns < ns_min) ns = ns_min;
    if (ns < 1) ns = 1;
    long c = (Skv + ns - 1) / ns;
    c = (c + 63) / 64 * 64;
    *chunk = (int)c;
    *nsplit = (int)((Skv + c - 1) / c);
}

size_t decode_workspace_bytes(int B, int H, int D, int nsplit) {
    if (nsplit <= 1) return 0;
    return (size_t)B * H * nsplit * (size_t)(D + 2) * sizeof(float);
}

// ---- element helpers ---------------------------------------------------------------------------

template <typename T>
struct Vec8;  // 8 consecutive 16-bit elements in four 32-bit registers

template <>
struct Vec8<half_t> {
    uint4_t r;
    __device__ __forceinline__ float dot(const Vec8 &o, float acc) const {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // copy the lane out first: bit-casting a vector-element lvalue reads element 0
            const uint32_t ra = r[i], rb = o.r[i];
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, ra), __builtin_bit_cast(half2_t, rb), acc, false);
        }
        return acc;
    }
    __device__ __forceinline__ float get(int e) const {
        const half8_t a = __builtin_bit_cast(half8_t, r);  // folds into v_fma_mix_f32 operand selects
        return (float)a[e];
    }
};

template <>
struct Vec8<bf16_t> {
    uint4_t r;
    __device__ __forceinline__ float get(int e) const {
        typedef uint16_t ushort8_t __attribute__((ext_vector_type(8)));
        const ushort8_t a = __builtin_bit_cast(ushort8_t, r);
        return __uint_as_float((uint32_t)a[e] << 16);
    }
    __device__ __forceinline__ float dot(const Vec8 &o, float acc) const {
#pragma unroll
        for (int e = 0; e < 8; e++) acc = fmaf(get(e), o.get(e), acc);
        return acc;
    }
};

template <int LPK>
__device__ __forceinline__ float lpk_sum(float x) {
    if constexpr (LPK == 16) return group_sum16(x);
    else if constexpr (LPK == 8) return group_sum8(x);
    else return group_sum4(x);
}

// ---- pass 1 -------------------------------------------------------------------------------------

template <typename T, int LPK, int GT>
__global__ __launch_bounds__(64 * DEC_WAVES) void decode_splitkv_kernel(AttnParams p) {
    constexpr int KPI = 64 / LPK;   // key rows covered by one wavefront load
    constexpr int U = DEC_UNROLL;
    constexpr int DMAX = LPK * 8;
    __shared__ float lds_acc[DEC_WAVES][GT][DMAX];
    __shared__ float lds_ml[DEC_WAVES][GT][2];

    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int r = lane / LPK;
    const int c = lane % LPK;
    const int D = p.D;
    const bool active = c * 8 < D;

    const int split = blockIdx.x;
    const int HB = (p.G + GT - 1) / GT;
    const int hb = blockIdx.y % HB;
    const int bg = blockIdx.y / HB;
    const int g = bg % p.Hkv;
    const int b = bg / p.Hkv;
    const int h0 = g * p.G + hb * GT;            // first query head of this block
    const int nh = min(GT, p.G - hb * GT);       // real heads in this block

    // visible key range of this workgroup
    int kv_hi = p.Skv;
    if (p.kv_lens) {
        const int len = p.kv_lens[b];
        kv_hi = min(kv_hi, max(len, 0));
    }
    if (p.kv_lens && split * p.chunk >= kv_hi && split > 0) return;  // beyond this sequence: the combine skips it
    int lo = split * p.chunk;
    int hi = min(lo + p.chunk, kv_hi);
    if (p.analytic) {
        if (p.causal) hi = (int)min((int64_t)hi, p.q_pos_offset + 1);
        if (p.window > 0) lo = (int)max((int64_t)lo, p.q_pos_offset - p.window + 1);
    }

    // query rows of the GT heads: the 8 elements this lane owns
    Vec8<T> q[GT];
#pragma unroll
    for (int hh = 0; hh < GT; hh++) {
        const int h = h0 + min(hh, nh - 1);
        const uint16_t *qp = (const uint16_t *)p.q + b * p.qs[0] + h * p.qs[1];
        uint32_t w[4] = {0, 0, 0, 0};
        if (active) {
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const uint32_t x = qp[(int64_t)(c * 8 + e) * p.qs[3]];
                w[e >> 1] |= x << ((e & 1) * 16);
            }
        }
        q[hh].r = uint4_t{w[0], w[1], w[2], w[3]};
    }

    const uint16_t *kbase = (const uint16_t *)p.k + b * p.ks[0] + g * p.ks[1] + c * 8;
    const uint16_t *vbase = (const uint16_t *)p.v + b * p.vs[0] + g * p.vs[1] + c * 8;
    const T *mrow = nullptr;
    if (p.mask_kind == FHIP_MASK_QK) mrow = (const T *)p.mask;
    if (p.mask_kind == FHIP_MASK_BATCH_KEY) mrow = (const T *)p.mask + b * p.ms0;
    const float scale2 = p.scale * LOG2E;

    float m[GT], l[GT], acc[GT][8];
#pragma unroll
    for (int hh = 0; hh < GT; hh++) {
        m[hh] = -INFINITY;
        l[hh] = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[hh][e] = 0.0f;
    }

    // keys of one workgroup step: (u, wave, r) -> lo_al + ((it*U + u) * DEC_WAVES + wave) * KPI + r
    const int lo_al = lo - (lo % (DEC_WAVES * KPI));
    for (int base = lo_al; base < hi; base += U * DEC_WAVES * KPI) {
        Vec8<T> kk[U], vv[U];
        int key[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            key[u] = base + (u * DEC_WAVES + wave) * KPI + r;
            const bool ok = active && key[u] >= lo && key[u] < hi;
            kk[u].r = uint4_t{0, 0, 0, 0};
            vv[u].r = uint4_t{0, 0, 0, 0};
            if (ok) {
                kk[u].r = *(const uint4_t *)(kbase + (int64_t)key[u] * p.ks[2]);
                vv[u].r = *(const uint4_t *)(vbase + (int64_t)key[u] * p.vs[2]);
            }
        }
        float s[U][GT];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const bool visible = key[u] >= lo && key[u] < hi;
            float bias = 0.0f;
            if (mrow && visible) bias = to_float(mrow[(int64_t)key[u] * p.ms1]) * LOG2E;
#pragma unroll
            for (int hh = 0; hh < GT; hh++) {
                float d = lpk_sum<LPK>(kk[u].dot(q[hh], 0.0f));
                d = d * scale2 + bias;
                s[u][hh] = visible ? d : -INFINITY;
            }
        }
#pragma unroll
        for (int hh = 0; hh < GT; hh++) {
            float mx = s[0][hh];
#pragma unroll
            for (int u = 1; u < U; u++) mx = fmaxf(mx, s[u][hh]);
            const float m_new = fmaxf(m[hh], mx);
            const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
            const float corr = exp2f(m[hh] - m_safe);
            float pu[U];
            float psum = 0.0f;
#pragma unroll
            for (int u = 0; u < U; u++) {
                pu[u] = exp2f(s[u][hh] - m_safe);
                psum += pu[u];
            }
            l[hh] = l[hh] * corr + psum;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                float a = acc[hh][e] * corr;
#pragma unroll
                for (int u = 0; u < U; u++) a = fmaf(pu[u], vv[u].get(e), a);
                acc[hh][e] = a;
            }
            m[hh] = m_new;
        }
    }

    // merge the KPI lane groups of this wavefront (lanes l, l ^ LPK, l ^ 2 LPK, ...)
#pragma unroll
    for (int off = LPK; off < 64; off <<= 1) {
#pragma unroll
        for (int hh = 0; hh < GT; hh++) {
            const float mo = __shfl_xor(m[hh], off, 64);
            const float lo_ = __shfl_xor(l[hh], off, 64);
            const float M = fmaxf(m[hh], mo);
            const float Ms = (M == -INFINITY) ? 0.0f : M;
            const float wa = exp2f(m[hh] - Ms), wb = exp2f(mo - Ms);
            l[hh] = l[hh] * wa + lo_ * wb;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float ao = __shfl_xor(acc[hh][e], off, 64);
                acc[hh][e] = acc[hh][e] * wa + ao * wb;
            }
            m[hh] = M;
        }
    }
    if (r == 0 && active) {
#pragma unroll
        for (int hh = 0; hh < GT; hh++) {
#pragma unroll
            for (int e = 0; e < 8; e++) lds_acc[wave][hh][c * 8 + e] = acc[hh][e];
            if (c == 0) {
                lds_ml[wave][hh][0] = m[hh];
                lds_ml[wave][hh][1] = l[hh];
            }
        }
    }
    __syncthreads();

    // merge the four wavefronts; thread t owns (head hh, dim d)
    for (int idx = threadIdx.x; idx < GT * DMAX; idx += 64 * DEC_WAVES) {
        const int hh = idx / DMAX, d = idx % DMAX;
        if (hh >= nh || d >= D) continue;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; w++) M = fmaxf(M, lds_ml[w][hh][0]);
        const float Ms = (M == -INFINITY) ? 0.0f : M;
        float L = 0.0f, A = 0.0f;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; w++) {
            const float wgt = exp2f(lds_ml[w][hh][0] - Ms);
            L += wgt * lds_ml[w][hh][1];
            A += wgt * lds_acc[w][hh][d];
        }
        const int h = h0 + hh;
        if (p.nsplit == 1) {
            const float o = A / L;  // no visible key: 0/0 = NaN like the reference
            const int64_t oi = b * p.os[0] + h * p.os[1] + d * p.os[3];
            if (p.out_f32) ((float *)p.out)[oi] = o;
            else ((T *)p.out)[oi] = from_float<T>(o);
        } else {
            float *ws = (float *)p.workspace + (((int64_t)b * p.H + h) * p.nsplit + split) * (D + 2);
            ws[d] = A;
            if (d == 0) {
                ws[D] = M;
                ws[D + 1] = L;
            }
        }
    }
}

// ---- pass 2 -------------------------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(64) void decode_combine_kernel(AttnParams p) {
    const int bh = blockIdx.x;
    const int h = bh % p.H, b = bh / p.H;
    const int D = p.D;
    int ns = p.nsplit;
    if (p.kv_lens) {
        const int len = min(p.Skv, max(p.kv_lens[b], 0));
        ns = max(1, min(ns, (len + p.chunk - 1) / p.chunk));  // split 0 is always written
    }
    const float *ws = (const float *)p.workspace + ((int64_t)b * p.H + h) * p.nsplit * (D + 2);
    float M = -INFINITY;
    for (int s = 0; s < ns; s++) M = fmaxf(M, ws[(int64_t)s * (D + 2) + D]);
    const float Ms = (M == -INFINITY) ? 0.0f : M;
    float L = 0.0f;
    for (int s = 0; s < ns; s++) L += exp2f(ws[(int64_t)s * (D + 2) + D] - Ms) * ws[(int64_t)s * (D + 2) + D + 1];
    for (int d = threadIdx.x; d < D; d += 64) {
        float A = 0.0f;
        for (int s = 0; s < ns; s++) A += exp2f(ws[(int64_t)s * (D + 2) + D] - Ms) * ws[(int64_t)s * (D + 2) + d];
        const float o = A / L;
        const int64_t oi = b * p.os[0] + h * p.os[1] + d * p.os[3];
        if (p.out_f32) ((float *)p.out)[oi] = o;
        else ((T *)p.out)[oi] = from_float<T>(o);
    }
}

template <typename T, int LPK>
static void launch_pass1(const AttnParams &p, dim3 grid, hipStream_t stream, int gt) {
    dim3 block(64 * DEC_WAVES);
    switch (gt) {
        case 1: hipLaunchKernelGGL((decode_splitkv_kernel<T, LPK, 1>), grid, block, 0, stream, p); break;
        case 2: hipLaunchKernelGGL((decode_splitkv_kernel<T, LPK, 2>), grid, block, 0, stream, p); break;
        case 4: hipLaunchKernelGGL((decode_splitkv_kernel<T, LPK, 4>), grid, block, 0, stream, p); break;
        default: hipLaunchKernelGGL((decode_splitkv_kernel<T, LPK, 8>), grid, block, 0, stream, p); break;
    }
}

template <typename T>
static int launch_decode_t(const AttnParams &p, hipStream_t stream) {
    const int gt = decode_gt(p.G);
    const int hb = (p.G + gt - 1) / gt;
    const long gy = (long)p.B * p.Hkv * hb;
    if (gy > 65535 || p.nsplit > 0x7fffffff) {
        set_error("decode: batch * kv_heads * head_blocks = %ld exceeds the grid limit 65535", gy);
        return FHIP_ERR_UNSUPPORTED;
    }
    dim3 grid((unsigned)p.nsplit, (unsigned)gy);
    if (p.D <= 32) launch_pass1<T, 4>(p, grid, stream, gt);
    else if (p.D <= 64) launch_pass1<T, 8>(p, grid, stream, gt);
    else launch_pass1<T, 16>(p, grid, stream, gt);
    FHIP_HIP_CHECK(hipGetLastError());
    if (p.main_done) FHIP_HIP_CHECK(hipEventRecord(p.main_done, stream));
    if (p.nsplit > 1) {
        hipLaunchKernelGGL(decode_combine_kernel<T>, dim3((unsigned)(p.B * p.H)), dim3(64), 0, stream, p);
        FHIP_HIP_CHECK(hipGetLastError());
    }
    return FHIP_OK;
}

int launch_decode(const AttnParams &p, fhip_dtype dtype, hipStream_t stream) {
    if (dtype == FHIP_F16) return launch_decode_t<half_t>(p, stream);
    if (dtype == FHIP_BF16) return launch_decode_t<bf16_t>(p, stream);
    set_error("decode kernel takes f16/bf16 only");
    return FHIP_ERR_UNSUPPORTED;
}

}  // namespace fhip
