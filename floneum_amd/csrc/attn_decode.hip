// Split-KV decode attention for a 16-bit KV cache (query length 1).
//
// Pass 1: grid = (split, batch * kv_head * head_block).  A workgroup of four wavefronts streams one
// chunk of keys/values of one KV head exactly once for all the query heads that share it (GQA
// group).  Two variants:
//   decode_mfma_kernel (head_dim 32/64/96/128): every wavefront load instruction reads 1 KB of
//     consecutive key (or value) rows with non-temporal 128-bit loads; the rows are parked in a
//     wavefront-private LDS tile and fed to the matrix cores: S^T[key][head] = K . Q^T with
//     v_mfma_f32_16x16x32 (the GQA heads, padded to 16, are the N dimension) and
//     O^T[dim][head] += V^T . P^T with V^T read by the transposing LDS load.  The softmax state of
//     head j lives in the lanes with lane % 16 == j, so scores, probabilities and the output
//     accumulator never change lanes.
//   decode_vec_kernel (any head_dim multiple of 8 up to 256): LPK lanes x 8 elements per row, dot
//     products on v_dot2, DPP reductions; every group of LPK lanes keeps its own softmax state.
// Both keep (m, l, acc) in the log2 domain, merge lanes -> wavefront -> workgroup at the end and
// write one partial (acc[D], m, l) per (batch, head, split).
// Pass 2 (decode_combine_kernel, decode_combine4_kernel): log-sum-exp merge of the partials of each (batch, head).
// With a single split pass 1 writes the final output and pass 2 is not launched.
//
// Reference semantics: fusor-ml/fusor/src/composite/flash_attention.rs:141-199 (f32 accumulation
// of 16-bit inputs as in fusor-ml/core/src/composite/flash_attention.rs:186-203,323-327).
#include <cstdlib>
#include <type_traits>

#include "common.h"
#include "device_utils.h"

namespace fhip {

constexpr int DEC_WAVES = 4;
constexpr int DEC_UNROLL = 4;
constexpr float LOG2E = 1.4426950408889634f;

// the matrix-core variants: 16-bit tensors on the 16-bit instruction at every multiple of 32 up to 256, f32 tensors on
// the f32 one likewise, except that at 224 and 256 a step of up to four columns per KV head (a plain decode step of a
// 4-way group) stays on the vector variant: the two are within 10 % of each other there, either way by shape, while
// with more columns the vector variant streams the cache once per query row (4 rows, B8 x 8192 keys, head_dim 256:
// 396 us against 110).  Above 128 one workgroup per CU, whose four wavefronts then have the registers and LDS of
// eight.  Other head dims run on the vector variant.  cols: (query head, query row) pairs of a KV head.
static bool decode_use_mfma(int D, bool f32, int cols) {
    if (!(D % 32 == 0 && D >= 32 && D <= 256)) return false;
    return !(f32 && D > 192 && cols <= 4);
}

// columns ((query head, query row) pairs of a KV head) handled by one workgroup: the matrix-core variants take one
// block of 16, or two when there are more than 16 columns: up to head_dim 128, and up to 192 for f32 tensors (f32, B8 x
// 8192 keys, 8 rows of a 4-way group at 192: 156 -> 115 us; at 256 the two blocks spill registers: 203 -> 291 us)
static int decode_gt(int G, int D, bool f32) {
    if (decode_use_mfma(D, f32, G)) return (G > 16 && D <= (f32 ? 192 : 128)) ? 32 : 16;
    return G <= 1 ? 1 : G <= 2 ? 2 : G <= 4 ? 4 : 8;
}

void decode_plan(int B, int Hkv, int G, int Skv, int D, int compute_units, bool ragged, bool f32, int *chunk,
                 int *nsplit, int *waves) {
    const int gt = decode_gt(G, D, f32);
    const int hb = (G + gt - 1) / gt;
    const long units = (long)B * Hkv * hb;
    *waves = DEC_WAVES;
    // The 8-wavefront form of the 16-bit matrix-core variant (one workgroup per CU).  With a whole (batch, KV head) unit
    // or more per CU: chunks of 2048 keys.  With more than 8 columns per unit (a multi-token step: twice the matrix and
    // softmax work per key) also below that, when an even share of the keys per CU is at least 2048 keys long: then
    // every CU gets one workgroup and all are equally long.
    if (decode_use_mfma(D, f32, G) && !f32 && D <= 128 && Skv > 2048) {
        if (units >= compute_units) {
            *waves = 8;
            *chunk = 2048;
            *nsplit = (Skv + 2047) / 2048;
            return;
        }
        const long ns = compute_units / units;  // >= 1
        const long c = ((Skv + ns - 1) / ns + 127) / 128 * 128;
        if (G > 8 && c >= 2048) {
            *waves = 8;
            *chunk = (int)c;
            *nsplit = (int)((Skv + c - 1) / c);
            return;
        }
    }
    // the MFMA variant holds two workgroups per CU (LDS; one above head_dim 128), the vector variant four or more; f32 rows carry
    // twice the bytes per workgroup step and do best with two as well (measured: +3 % at batch 16, +16 % at
    // batch 1 with 32768 keys)
    const int wgs_per_cu = (decode_use_mfma(D, f32, G) && D > 128) ? 1 : (decode_use_mfma(D, f32, G) || f32) ? 2 : 4;
    const long target = (long)compute_units * wgs_per_cu;
    // short chunks even out a ragged batch (measured: 512 beats 1024 by 12 % on a 128..32768-token
    // batch); with equal lengths the longer chunk is 2-3 % ahead
    const int max_chunk = ragged && units >= target ? 512 : 1024;
    // few (batch, kv head) units, e.g. batch 1: down to one workgroup step of 128 keys per split, because a
    // workgroup's steps run one after the other and each costs a memory latency.  Up to 256 keys the matrix-core
    // variant is quicker unsplit than with a second launch to merge two splits (measured 6.6 vs 8.6 us).
    // (the vector variant's step is 16 rows of 64 / LPK keys: 64 keys at head_dim 128 in f32, where one step
    // per workgroup is one memory round trip less than two)
    int step_keys = f32 ? 64 : 128;  // matrix-core variants: four wavefronts of 16 (f32) or 32 keys
    if (!decode_use_mfma(D, f32, G)) {
        const int lpk = D <= 32 ? 4 : D <= 64 ? 8 : D <= 128 ? 16 : 32;
        step_keys = 16 * (64 / lpk);
        if (step_keys > 128) step_keys = 128;
    }
    const int min_chunk = step_keys;
    long ns = (target + units - 1) / units;
    const long ns_max = (Skv + min_chunk - 1) / min_chunk;
    const long ns_min = (Skv + max_chunk - 1) / max_chunk;
    if (ns > ns_max) ns = ns_max;
    if (ns < ns_min) ns = ns_min;
    if (ns < 1 || (Skv <= 256 && decode_use_mfma(D, f32, G))) ns = 1;
    long c = (Skv + ns - 1) / ns;
    c = (c + step_keys - 1) / step_keys * step_keys;  // whole workgroup steps
    *chunk = (int)c;
    *nsplit = (int)((Skv + c - 1) / c);
}

// Workspace: the partials, B * H * nsplit * (D + 2) floats (H counts (head, row) pairs), plus what the fused merge adds:
// every split's partials start on a 128-byte line, and one arrival counter per unit behind them.
size_t decode_workspace_bytes(int B, int H, int Hkv, int D, int nsplit) {
    if (nsplit <= 1) return 0;
    // columns of a KV head, padded to whole column blocks of 16 or 32 where there is more than one block
    const size_t cols = (size_t)H / Hkv;
    size_t padded = cols;
    for (size_t gt = 16; gt <= 32; gt *= 2)
        if (cols > gt && (cols + gt - 1) / gt * gt > padded) padded = (cols + gt - 1) / gt * gt;
    const size_t units = (size_t)B * Hkv * ((cols + 15) / 16);
    const size_t partials = (size_t)B * Hkv * padded * nsplit * (size_t)(D + 2) * sizeof(float);
    if (nsplit > 8) return partials;  // never merged inside the main kernel
    return partials + units * ((size_t)nsplit * 128 + sizeof(uint32_t)) + 256;
}

// The fused merge (the matrix-core variants with p.dec_fused): 2 to 8 splits, equal lengths.
// *unit_stride: floats between the partials of consecutive units; *counters_offset: bytes from the workspace's start
// to the arrival counters.
bool decode_fused_layout(const AttnParams &p, bool f32, int *unit_stride, size_t *counters_offset) {
    const int cols = p.G * p.Sq;
    if (!decode_use_mfma(p.D, f32, cols) || p.nsplit < 2 || p.nsplit > 8 || p.kv_lens) return false;
    const int gt = decode_gt(cols, p.D, f32);
    const long units = (long)p.B * p.Hkv * ((cols + gt - 1) / gt);
    const long stride = p.nsplit * (((long)(cols < gt ? cols : gt) * (p.D + 2) + 31) / 32 * 32);
    if ((units + 7) / 8 * 8 * p.nsplit > 0x7fffffffL || stride > 0x7fffffffL) return false;
    *unit_stride = (int)stride;
    *counters_offset = ((size_t)units * stride * sizeof(float) + 255) & ~(size_t)255;
    return true;
}

// ---- element helpers ---------------------------------------------------------------------------

template <typename T>
struct Vec8;  // 8 consecutive elements of a row: four 32-bit registers for 16-bit types, eight for f32

// shared by the 16-bit specialisations
struct Vec8Bits16 {
    uint4_t r;
    __device__ __forceinline__ void zero() { r = uint4_t{0, 0, 0, 0}; }
    __device__ __forceinline__ void load(const void *p) { r = *(const uint4_t *)p; }
    // 8 elements `stride` apart (the query row, which may have any stride)
    __device__ __forceinline__ void gather(const void *p, int64_t stride) {
        const uint16_t *q = (const uint16_t *)p;
        uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < 8; e++) w[e >> 1] |= (uint32_t)q[e * stride] << ((e & 1) * 16);
        r = uint4_t{w[0], w[1], w[2], w[3]};
    }
};

template <>
struct Vec8<float> {
    float4_t a, b;
    __device__ __forceinline__ void zero() { a = b = float4_t{0.f, 0.f, 0.f, 0.f}; }
    __device__ __forceinline__ void load(const void *p) {
        a = *(const float4_t *)p;
        b = *((const float4_t *)p + 1);
    }
    __device__ __forceinline__ void gather(const void *p, int64_t stride) {
        const float *q = (const float *)p;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            a[e] = q[e * stride];
            b[e] = q[(e + 4) * stride];
        }
    }
    __device__ __forceinline__ float get(int e) const { return e < 4 ? a[e] : b[e - 4]; }
    __device__ __forceinline__ float dot(const Vec8 &o, float acc) const {
#pragma unroll
        for (int e = 0; e < 4; e++) acc = fmaf(a[e], o.a[e], acc);
#pragma unroll
        for (int e = 0; e < 4; e++) acc = fmaf(b[e], o.b[e], acc);
        return acc;
    }
};

template <>
struct Vec8<half_t> : Vec8Bits16 {
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
struct Vec8<bf16_t> : Vec8Bits16 {
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
    if constexpr (LPK == 32) return group_sum32(x);
    else if constexpr (LPK == 16) return group_sum16(x);
    else if constexpr (LPK == 8) return group_sum8(x);
    else return group_sum4(x);
}

// ---- pass 1 -------------------------------------------------------------------------------------

template <typename T, int LPK, int GT>
__global__ __launch_bounds__(64 * DEC_WAVES) void decode_vec_kernel(AttnParams p) {
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

    // Workgroups go to the 8 XCDs round-robin in launch order (x fastest), and with ragged lengths only the
    // first splits of a row of the grid have keys: taken as they come, XCD 0 would get up to one more busy
    // workgroup per (batch, head) than XCD 7.  Rotating the split by the row spreads them evenly.
    const int split = (int)((blockIdx.x + blockIdx.y) % (unsigned)p.nsplit);
    // A workgroup serves up to GT columns = (query head, query row) pairs that share the KV head: column c is head
    // c / rows, row c % rows of the group (one row per head in a plain decode step, a few in a multi-token step).
    const int rows = p.Sq;
    const int NC = p.G * rows;
    const int HB = (NC + GT - 1) / GT;
    const int hb = blockIdx.y % HB;
    const int bg = blockIdx.y / HB;
    const int g = bg % p.Hkv;
    const int b = bg / p.Hkv;
    const int c0 = hb * GT;                      // first column of this block
    const int nh = min(GT, NC - c0);             // columns in use

    // visible key range of this workgroup
    int kv_hi = p.Skv;
    if (p.kv_lens) {
        const int len = p.kv_lens[b];
        kv_hi = min(kv_hi, max(len, 0));
    }
    if (p.kv_lens && split * p.chunk >= kv_hi && split > 0) return;  // beyond this sequence: the combine skips it
    // [lo, hi): the keys some row sees.  Row r sees key j when j - r lies in [first, limit): the causal limit and the
    // start of the window move with the row (limits that do not apply are set out of reach).
    int lo = split * p.chunk;
    int hi = min(lo + p.chunk, kv_hi);
    int limit = 0x3fffffff, first = -0x3fffffff;
    if (p.analytic) {
        if (p.causal) {
            limit = (int)min((int64_t)limit, p.q_pos_offset + 1);
            hi = (int)min((int64_t)hi, p.q_pos_offset + rows);
        }
        if (p.window > 0) {
            first = (int)max((int64_t)first, p.q_pos_offset - p.window + 1);
            lo = max(lo, first);
        }
    }

    // query rows of the GT columns: the 8 elements this lane owns
    Vec8<T> q[GT];
    int rr[GT];  // query row of each column
#pragma unroll
    for (int hh = 0; hh < GT; hh++) {
        const int col = c0 + min(hh, nh - 1);
        const int h = g * p.G + col / rows;
        rr[hh] = col % rows;
        const T *qp = (const T *)p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)rr[hh] * p.qs[2];
        q[hh].zero();
        if (active) {
            // one 16 / 32-byte load when the row is contiguous and aligned, element by element otherwise
            if (p.qs[3] == 1 && (((uintptr_t)(qp + c * 8)) & 15) == 0) q[hh].load(qp + c * 8);
            else q[hh].gather(qp + (int64_t)(c * 8) * p.qs[3], p.qs[3]);
        }
    }

    const T *kbase = (const T *)p.k + b * p.ks[0] + g * p.ks[1] + c * 8;
    const T *vbase = (const T *)p.v + b * p.vs[0] + g * p.vs[1] + c * 8;
    const T *mrow = nullptr;
    if (p.mask_kind == FHIP_MASK_QK) mrow = (const T *)p.mask;
    if (p.mask_kind == FHIP_MASK_BATCH_KEY) mrow = (const T *)p.mask + b * p.ms0;
    const bool row_masks = rows > 1 && p.mask_kind == FHIP_MASK_QK;  // every query row has its own mask row
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
            kk[u].zero();
            vv[u].zero();
            if (ok) {
                kk[u].load(kbase + (int64_t)key[u] * p.ks[2]);
                vv[u].load(vbase + (int64_t)key[u] * p.vs[2]);
            }
        }
        float s[U][GT];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const bool visible = key[u] >= lo && key[u] < hi;
            float bias = 0.0f;
            if (mrow && visible && !row_masks) bias = to_float(mrow[(int64_t)key[u] * p.ms1]) * LOG2E;
#pragma unroll
            for (int hh = 0; hh < GT; hh++) {
                float d = lpk_sum<LPK>(kk[u].dot(q[hh], 0.0f));
                const int rel = key[u] - rr[hh];
                const bool vis = visible && rel < limit && rel >= first;
                float bh = bias;
                if (row_masks && vis) bh = to_float(mrow[(int64_t)rr[hh] * p.ms0 + (int64_t)key[u] * p.ms1]) * LOG2E;
                d = d * scale2 + bh;
                s[u][hh] = vis ? d : -INFINITY;
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
        const int h = g * p.G + (c0 + hh) / rows, qr = (c0 + hh) % rows;
        if (p.nsplit == 1) {
            const float o = A / L;  // no visible key: 0/0 = NaN like the reference
            const int64_t oi = b * p.os[0] + h * p.os[1] + qr * p.os[2] + d * p.os[3];
            if (p.out_f32) ((float *)p.out)[oi] = o;
            else ((T *)p.out)[oi] = from_float<T>(o);
        } else {
            float *ws = (float *)p.partials + ((((int64_t)b * p.H + h) * rows + qr) * p.nsplit + split) * (D + 2);
            ws[d] = A;
            if (d == 0) {
                ws[D] = M;
                ws[D + 1] = L;
            }
        }
    }
}

// ---- pass 1, matrix-core variant ----------------------------------------------------------------------

#define DLDS_PTR(type, byte_off) ((__attribute__((address_space(3))) type *)(lds_base + (byte_off)))

typedef uint32_t uint2v_t __attribute__((ext_vector_type(2)));

template <typename T>
struct DecMma;
template <>
struct DecMma<half_t> {
    typedef half8_t vec8;
    static __device__ __forceinline__ float4_t mfma(vec8 a, vec8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float x, float y) {
        half2_t h = {(half_t)x, (half_t)y};
        return __builtin_bit_cast(uint32_t, h);
    }
};
template <>
struct DecMma<bf16_t> {
    typedef bf16x8_t vec8;
    static __device__ __forceinline__ float4_t mfma(vec8 a, vec8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float x, float y) {
        return (uint32_t)from_float<bf16_t>(x).bits | ((uint32_t)from_float<bf16_t>(y).bits << 16);
    }
};

// max / sum over the four lanes l, l^16, l^32, l^48 (same head, the four key groups)
__device__ __forceinline__ float quad_rows_max(float x) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float quad_rows_sum(float x) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// ---- fused merge of the matrix-core variants ----------------------------------------------------------------------
// With p.dec_fused the launch is one-dimensional and the workgroups of a (batch, kv head, column block) unit are
// numbered so that they run on ONE XCD: the hardware deals the workgroups of a launch to its XCDs round-robin in launch
// order (workgroup L + 1 runs on the XCD after workgroup L's; where workgroup 0 lands depends on what the queue ran
// before), so workgroups with the same L % 8 share an XCD whether the device has 8, 4, 2 or 1 of them (checked per
// device before the form is ever chosen).  Their partials then meet in that XCD's L2 and the last workgroup of the unit
// to arrive merges them: no second kernel, whose dependent launch costs a few microseconds (batch 16 x 4096 keys, f16:
// 47.1 -> 46.3 us per step; head_dim 256: 54.3 -> 52.2).  The arrival counter itself is kept coherent over the whole
// device (with partials AND counter device-coherent the form is slower than two kernels) and carries the XCC id of the
// first workgroup to arrive: a workgroup that arrives from another XCD sets the host-visible word p.dec_trip, which
// fails the device's next decode call and switches the form off.
__device__ __forceinline__ uint32_t xcc_id() {
    uint32_t x;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
    return x & 15u;
}

__global__ void xcd_probe_kernel(uint8_t *out) {
    if (threadIdx.x == 0) out[blockIdx.x] = (uint8_t)xcc_id();
}

int launch_xcd_probe(uint8_t *out, int workgroups, hipStream_t stream) {
    hipLaunchKernelGGL(xcd_probe_kernel, dim3((unsigned)workgroups), dim3(64), 0, stream, out);
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

// unit and split of this workgroup (false: the launch is padded to a multiple of 8 units and this one is beyond the end)
__device__ __forceinline__ bool decode_unit_of_workgroup(const AttnParams &p, int units, int *unit, int *split) {
    if (p.dec_fused) {
        const unsigned xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
        *split = (int)(slot % (unsigned)p.nsplit);
        *unit = (int)(slot / (unsigned)p.nsplit) * 8 + (int)xcd;
        return *unit < units;
    }
    // spread the splits over the XCDs, see decode_vec_kernel
    *split = (int)((blockIdx.x + blockIdx.y) % (unsigned)p.nsplit);
    *unit = blockIdx.y;
    return true;
}

// where a workgroup parks column hh of its split in the fused form: a unit's partials are [split][column][D + 2], and
// every split's part starts on a 128-byte line of its own (no line is written by two workgroups)
__device__ __forceinline__ float *fused_partial_row(const AttnParams &p, int unit, int split, int hh, int D) {
    return (float *)p.partials + (int64_t)unit * p.dec_unit_stride + split * (p.dec_unit_stride / p.nsplit) + hh * (D + 2);
}

// After every thread of the workgroup has stored its part of the unit's partials: count the arrival; the last
// workgroup of the unit merges the splits in order with the arithmetic of decode_combine_kernel (same bits) and
// writes the output rows.  Every access is served by this XCD's L2: the stores have been acknowledged by it before
// the arrival is counted (an atomic in the same L2), and the last workgroup reads lines nobody on its CU has read in
// this launch (every split's partials have whole lines to themselves, one writer and one reader).  Nothing spins: a workgroup that
// is not the last leaves.  The counter holds (tag << 8) | arrivals with a tag unique to the call, so it needs no
// clearing: whatever else it holds (another call's count, the finished count of a replay of this call) restarts it.
template <typename T, int THREADS>
__device__ __forceinline__ void fused_merge_tail(const AttnParams &p, int unit, int nh, int D, int b, int g, int c0, int rows) {
    __shared__ int is_last;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        // word: tag (20 bits) | XCC id of the first workgroup to arrive (4) | arrivals (8)
        uint32_t *ctr = p.dec_counters + unit;
        const uint32_t tag = p.dec_tag & 0xfffffu, xcc = xcc_id();
        const uint32_t fresh = (tag << 12) | (xcc << 8) | 1u;
        uint32_t cur = (tag << 12) | (xcc << 8), want;
        do {
            want = ((cur >> 12) == tag && (cur & 255u) < (uint32_t)p.nsplit) ? cur + 1 : fresh;
        } while (!__hip_atomic_compare_exchange_strong(ctr, &cur, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT));
        // the count is kept coherent over the whole device, so a unit whose workgroups are NOT on one XCD is seen here
        if (((want >> 8) & 15u) != xcc) __hip_atomic_store(p.dec_trip, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        is_last = (want & 255u) == (uint32_t)p.nsplit;
    }
    __syncthreads();
    if (!is_last) return;
    const float *wu = (const float *)p.partials + (int64_t)unit * p.dec_unit_stride;
    const int split_stride = p.dec_unit_stride / p.nsplit;
    for (int idx = threadIdx.x; idx < nh * D; idx += THREADS) {
        const int hh = idx / D, d = idx % D;
        float ms[8], ls[8], as[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const bool ok = u < p.nsplit;
            const float *src = wu + (ok ? u : 0) * split_stride + hh * (D + 2);
            ms[u] = ok ? src[D] : -INFINITY;
            ls[u] = ok ? src[D + 1] : 0.0f;
            as[u] = ok ? src[d] : 0.0f;
        }
        float Mn = -INFINITY;
#pragma unroll
        for (int u = 0; u < 8; u++) Mn = fmaxf(Mn, ms[u]);
        const float Ms = (Mn == -INFINITY) ? 0.0f : Mn;
        float L = 0.0f, A = 0.0f;
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const float w = __builtin_amdgcn_exp2f(ms[u] - Ms);
            L += w * ls[u];
            A += w * as[u];
        }
        const int h = g * p.G + (c0 + hh) / rows, qr = (c0 + hh) % rows;
        const float val = A / L;  // no visible key: 0/0 = NaN like the reference
        const int64_t oi = b * p.os[0] + h * p.os[1] + qr * p.os[2] + d * p.os[3];
        if (p.out_f32) ((float *)p.out)[oi] = val;
        else ((T *)p.out)[oi] = from_float<T>(val);
    }
}

constexpr int DM_KEYS = 32;  // keys per wavefront step
constexpr int DM_DEPTH = 1;  // tiles in flight per wavefront beside the one in LDS (2 measured no faster: the stream
                             // is not latency-bound with eight wavefronts per CU)
constexpr int DM_HEADS = 16; // query heads per workgroup (MFMA N dimension)

// WAVES = 4: two workgroups per CU.  WAVES = 8: one workgroup per CU with chunks of up to 2048 keys, for calls with at
// least one (batch, kv head) unit per CU: a workgroup's first tile takes several microseconds to arrive while the
// memory system is loaded, so with work enough to keep every CU busy anyway, fewer and longer workgroups stream
// better (32 ragged sequences of up to 32768 keys: 6.45 -> 6.83 TB/s).
// CB: 16-column blocks per workgroup.  With two, the K and V tiles a wavefront has parked in LDS serve 32 columns (a
// multi-token step with up to 32 (query head, query row) pairs per KV head): every LDS operand read feeds a matrix step
// for each block, and each block keeps its own softmax state.
template <typename T, int D, int WAVES, int CB>
__global__ __launch_bounds__(64 * WAVES, D > 128 ? 1 : 8 / WAVES) void decode_mfma_kernel(AttnParams p) {
    typedef typename DecMma<T>::vec8 vec8;
    constexpr int KP = D * 2 + 16;          // K tile row pitch (bytes): rows 4 banks apart
    constexpr int VP = D * 2 + 32;          // V tile row pitch (bytes): rows 8 banks apart
    constexpr int K_BYTES = DM_KEYS * KP;
    constexpr int V_BYTES = DM_KEYS * VP;
    constexpr int WAVE_BYTES = K_BYTES + V_BYTES;
    constexpr int CPR = D / 8;              // 16-byte chunks per row
    constexpr int NLD = DM_KEYS * CPR / 64; // 16-byte loads per lane per tile
    constexpr int KB = D / 32;              // contraction blocks of QK^T
    constexpr int NB = D / 16;              // 16-dim blocks of the output
    constexpr int COLS = DM_HEADS * CB;     // columns per workgroup
    constexpr int MERGE_BYTES = WAVES * COLS * (D + 2) * 4;
    constexpr int LDS_BYTES = WAVES * WAVE_BYTES > MERGE_BYTES ? WAVES * WAVE_BYTES : MERGE_BYTES;
    __shared__ __attribute__((aligned(16))) char smem[LDS_BYTES];

    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int j = lane & 15;  // column of this lane inside each block
    const int q4 = lane >> 4; // key group
    auto lds_base = (__attribute__((address_space(3))) char *)smem + wave * WAVE_BYTES;

    // The MFMA columns are the (query head, query row) pairs that share this KV head: column c is head c / rows,
    // row c % rows of the group (one row per head in a plain decode step, a few in a multi-token step).
    const int rows = p.Sq;
    const int NC = p.G * rows;
    const int HB = (NC + COLS - 1) / COLS;
    int split, unit;
    if (!decode_unit_of_workgroup(p, p.B * p.Hkv * HB, &unit, &split)) return;
    const int hb = unit % HB;
    const int bg = unit / HB;
    const int g = bg % p.Hkv;
    const int b = bg / p.Hkv;
    const int c0 = hb * COLS;
    const int nh = min(COLS, NC - c0);  // columns in use
    int hj[CB], rj[CB];                 // head and row of this lane's column in block cb
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        const int cj = c0 + min(j + DM_HEADS * cb, nh - 1);
        hj[cb] = g * p.G + cj / rows, rj[cb] = cj % rows;
    }

    int kv_hi = p.Skv;
    if (p.kv_lens) kv_hi = min(kv_hi, max(p.kv_lens[b], 0));
    if (p.kv_lens && split * p.chunk >= kv_hi && split > 0) return;  // the combine pass skips it too
    // [lo, hi): the keys some row of the workgroup sees; [lo_j, hi_j): the keys this lane's row sees
    int lo = split * p.chunk;
    int hi = min(lo + p.chunk, kv_hi);
    int lo_j[CB], hi_j[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        lo_j[cb] = lo, hi_j[cb] = hi;
        if (p.analytic && p.causal) hi_j[cb] = (int)min((int64_t)hi, p.q_pos_offset + 1 + rj[cb]);
        if (p.analytic && p.window > 0) lo_j[cb] = (int)max((int64_t)lo, p.q_pos_offset - p.window + 1 + rj[cb]);
    }
    if (p.analytic) {
        if (p.causal) hi = (int)min((int64_t)hi, p.q_pos_offset + rows);                // the last row sees furthest
        if (p.window > 0) lo = (int)max((int64_t)lo, p.q_pos_offset - p.window + 1);    // the first row sees the earliest key
    }

    const uint16_t *kbase = (const uint16_t *)p.k + b * p.ks[0] + g * p.ks[1];
    const uint16_t *vbase = (const uint16_t *)p.v + b * p.vs[0] + g * p.vs[1];
    const T *mrow[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        mrow[cb] = nullptr;
        if (p.mask_kind == FHIP_MASK_QK) mrow[cb] = (const T *)p.mask + rj[cb] * p.ms0;
        if (p.mask_kind == FHIP_MASK_BATCH_KEY) mrow[cb] = (const T *)p.mask + b * p.ms0;
    }
    const bool has_mask = p.mask_kind != FHIP_MASK_NONE;
    const float scale2 = p.scale * LOG2E;

    float4_t o[CB][NB];
    float m[CB], l[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) o[cb][nb] = float4_t{0.f, 0.f, 0.f, 0.f};
        m[cb] = -INFINITY, l[cb] = 0.0f;
    }

    // one wavefront step = 32 consecutive keys; the four wavefronts interleave their steps
    const int lo_al = lo - (lo % DM_KEYS);
    const int step = WAVES * DM_KEYS;
    // Staging registers of the tiles in flight: DEPTH tiles per wavefront.
    // Every lane always loads: a row outside [lo, hi) is replaced by the nearest one inside (its score is set to
    // -inf below, so what it holds never counts).  Without branches around the loads the compiler can count them,
    // and the wait in front of an LDS store is for that tile's loads only, not for everything in flight.
    constexpr int DEPTH = DM_DEPTH;
    uint4_t kst[DEPTH][NLD], vst[DEPTH][NLD];
    auto load_tile = [&](int base, auto set) __attribute__((always_inline)) {
        constexpr int S = decltype(set)::value;
#pragma unroll
        for (int u = 0; u < NLD; u++) {
            const int cid = lane + 64 * u;
            const int row = cid / CPR, col = cid % CPR;
            const int key = min(max(base + row, lo), hi - 1);
            kst[S][u] = __builtin_nontemporal_load((const uint4_t *)(kbase + (int64_t)key * p.ks[2] + col * 8));
            vst[S][u] = __builtin_nontemporal_load((const uint4_t *)(vbase + (int64_t)key * p.vs[2] + col * 8));
        }
    };
    auto store_tile = [&](auto set) __attribute__((always_inline)) {
        constexpr int S = decltype(set)::value;
#pragma unroll
        for (int u = 0; u < NLD; u++) {
            const int cid = lane + 64 * u;
            const int row = cid / CPR, col = cid % CPR;
            *DLDS_PTR(uint4_t, row * KP + col * 16) = kst[S][u];
            *DLDS_PTR(uint4_t, K_BYTES + row * VP + col * 16) = vst[S][u];
        }
    };
    using set0 = std::integral_constant<int, 0>;
    using set1 = std::integral_constant<int, DEPTH - 1>;

    int base = lo_al + wave * DM_KEYS;
    if (base < hi) {  // issued first so the Q fetch below overlaps them
        load_tile(base, set0{});
        if constexpr (DEPTH == 2) load_tile(base + step, set1{});
    }

    // Q^T operand: column j, dims 32 kb + 8 q4 .. +8 (zero for the padding columns)
    vec8 qreg[CB][KB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        const uint16_t *qp = (const uint16_t *)p.q + b * p.qs[0] + (int64_t)hj[cb] * p.qs[1] + (int64_t)rj[cb] * p.qs[2];
        const bool qvec = p.qs[3] == 1 && (((uintptr_t)qp) & 15) == 0;
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
            uint4_t raw = {0, 0, 0, 0};
            if (j + DM_HEADS * cb < nh) {
                if (qvec) {
                    raw = *(const uint4_t *)(qp + 32 * kb + 8 * q4);
                } else {
                    uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        const uint32_t x = qp[(int64_t)(32 * kb + 8 * q4 + e) * p.qs[3]];
                        w[e >> 1] |= x << ((e & 1) * 16);
                    }
                    raw = uint4_t{w[0], w[1], w[2], w[3]};
                }
            }
            qreg[cb][kb] = __builtin_bit_cast(vec8, raw);
        }
    }

    // one step: the staged tile `set` (keys base ..) goes to LDS, its registers take the tile DEPTH steps ahead, then the math
    auto one_step = [&](int base, auto set) __attribute__((always_inline)) {
        wave_lds_sync();  // the previous step's LDS reads precede these writes
        store_tile(set);
        wave_lds_sync();
        load_tile(base + DEPTH * step, set);  // in flight during the math below (beyond the end: a row read again)

        // ---- S^T[key][col] = K . Q^T : two 16-key tiles, every K operand read serves all column blocks -------
        float4_t s[CB][2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
#pragma unroll
            for (int cb = 0; cb < CB; cb++) s[cb][t] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kb = 0; kb < KB; kb++) {
                const uint4_t raw = *DLDS_PTR(uint4_t, (16 * t + j) * KP + (32 * kb + 8 * q4) * 2);
#pragma unroll
                for (int cb = 0; cb < CB; cb++)
                    s[cb][t] = DecMma<T>::mfma(__builtin_bit_cast(vec8, raw), qreg[cb][kb], s[cb][t]);
            }
        }
        vec8 pop[CB];
#pragma unroll
        for (int cb = 0; cb < CB; cb++) {
            // element (t, r) is key base + 16 t + 4 q4 + r for column j of block cb
            float sv[8];
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int key = base + 16 * t + 4 * q4 + r;
                    const bool visible = key >= lo_j[cb] && key < hi_j[cb];
                    float x = s[cb][t][r] * scale2;
                    if (has_mask && visible) x += to_float(mrow[cb][(int64_t)key * p.ms1]) * LOG2E;
                    sv[4 * t + r] = visible ? x : -INFINITY;
                }
            float mx = sv[0];
#pragma unroll
            for (int e = 1; e < 8; e++) mx = fmaxf(mx, sv[e]);
            mx = quad_rows_max(mx);
            const float m_new = fmaxf(m[cb], mx);
            const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
            const float corr = __builtin_amdgcn_exp2f(m[cb] - m_safe);
            m[cb] = m_new;
            float pe[8], psum = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                pe[e] = __builtin_amdgcn_exp2f(sv[e] - m_safe);
                psum += pe[e];
            }
            l[cb] = l[cb] * corr + psum;
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
                for (int r = 0; r < 4; r++) o[cb][nb][r] *= corr;
            // P^T operand: contraction slot (q4, e) is key 4 q4 + e (e < 4) or 16 + 4 q4 + e - 4
            const uint4_t praw = {DecMma<T>::pack2(pe[0], pe[1]), DecMma<T>::pack2(pe[2], pe[3]),
                                  DecMma<T>::pack2(pe[4], pe[5]), DecMma<T>::pack2(pe[6], pe[7])};
            pop[cb] = __builtin_bit_cast(vec8, praw);
        }

        // ---- O^T[dim][col] += V^T . P^T -----------------------------------------------------------------
        // the transposing load hands lane i of a 16-lane block V[row0 + 0..3][dim0 + i]; the lane
        // supplies the address of row0 + i / 4, dims dim0 + 4 (i % 4)
        const int trow = 4 * q4 + (j >> 2);
        const int tcol = 4 * (j & 3) * 2;
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const short4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                DLDS_PTR(short4_t, K_BYTES + trow * VP + nb * 32 + tcol));
            const short4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                DLDS_PTR(short4_t, K_BYTES + (16 + trow) * VP + nb * 32 + tcol));
            const uint2v_t u0 = __builtin_bit_cast(uint2v_t, a0), u1 = __builtin_bit_cast(uint2v_t, a1);
            const uint4_t araw = {u0[0], u0[1], u1[0], u1[1]};
#pragma unroll
            for (int cb = 0; cb < CB; cb++)
                o[cb][nb] = DecMma<T>::mfma(__builtin_bit_cast(vec8, araw), pop[cb], o[cb][nb]);
        }
    };
    for (; base < hi; base += DEPTH * step) {
        one_step(base, set0{});
        if constexpr (DEPTH == 2)
            if (base + step < hi) one_step(base + step, set1{});
    }

    // ---- merge: key groups -> wavefront -> workgroup ------------------------------------------------
    __syncthreads();  // every wavefront is done with its K/V tile; the LDS is reused for the merge
    float *macc = (float *)smem;  // [wave][column][D + 2]
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        const float l_col = quad_rows_sum(l[cb]);
        if (j + DM_HEADS * cb < nh) {
            float *dst = macc + ((wave * COLS + j + DM_HEADS * cb) * (D + 2));
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
                for (int r = 0; r < 4; r++) dst[16 * nb + 4 * q4 + r] = o[cb][nb][r];
            if (q4 == 0) {
                dst[D] = m[cb];
                dst[D + 1] = l_col;
            }
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < nh * D; idx += 64 * WAVES) {
        const int hh = idx / D, d = idx % D;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; w++) M = fmaxf(M, macc[(w * COLS + hh) * (D + 2) + D]);
        const float Ms = (M == -INFINITY) ? 0.0f : M;
        float L = 0.0f, A = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) {
            const float *src = macc + (w * COLS + hh) * (D + 2);
            const float wgt = __builtin_amdgcn_exp2f(src[D] - Ms);
            L += wgt * src[D + 1];
            A += wgt * src[d];
        }
        const int h = g * p.G + (c0 + hh) / rows, qr = (c0 + hh) % rows;
        if (p.nsplit == 1) {
            const float val = A / L;  // no visible key: 0/0 = NaN like the reference
            const int64_t oi = b * p.os[0] + h * p.os[1] + qr * p.os[2] + d * p.os[3];
            if (p.out_f32) ((float *)p.out)[oi] = val;
            else ((T *)p.out)[oi] = from_float<T>(val);
        } else {
            float *ws = p.dec_fused
                            ? fused_partial_row(p, unit, split, hh, D)
                            : (float *)p.partials + ((((int64_t)b * p.H + h) * rows + qr) * p.nsplit + split) * (D + 2);
            ws[d] = A;
            if (d == 0) {
                ws[D] = M;
                ws[D + 1] = L;
            }
        }
    }
    if (p.dec_fused && p.nsplit > 1) fused_merge_tail<T, 64 * WAVES>(p, unit, nh, D, b, g, c0, rows);
}

// ---- pass 1, matrix-core variant for f32 tensors -------------------------------------------------------
// The cache type kalosm-llama keeps (models/kalosm-llama/src/raw/attention_layer.rs:400-403).  Same structure as
// decode_mfma_kernel on v_mfma_f32_16x16x4_f32 (full f32 products): a wavefront step is 16 consecutive keys, parked
// in a wavefront-private LDS tile.
//   S^T[key][col] = K . Q^T : lane (j, q4) reads K[key j][16 c + 4 q4 .. +4] with one 128-bit LDS read per chunk c and
//     feeds its four values to four matrix steps (contraction slot (c, i, q4) = dim 16 c + 4 q4 + i on both operands);
//     the lane ends up with the scores of keys 4 q4 + r (r = 0..3) for column j.
//   O^T[dim][col] += V^T . P^T : contraction slot (ks, q4) is key 4 q4 + ks, so the B operand of step ks is the lane's
//     own probability r = ks (nothing changes lanes).  Lane (i, q4) reads VW consecutive dims of V[key 4 q4 + ks] with
//     one LDS read and feeds VW matrix steps: row i of output block (hb, e) is dim 16 VW hb + VW i + e.  The lane
//     therefore holds, for its column, the 4 VW consecutive dims starting at 16 VW hb + 4 VW q4 of every block hb.
// The vector variant spends most of its instructions on a softmax that every lane of a key's group repeats; here
// the softmax of a column is computed once, by the four lanes that hold its 16 scores.
constexpr int DF_KEYS = 16;  // keys per wavefront step

template <int D, int CB>  // CB: 16-column blocks per workgroup, see decode_mfma_kernel
__global__ __launch_bounds__(64 * DEC_WAVES, D > 128 ? 1 : 2) void decode_mfma_f32_kernel(AttnParams p) {
    constexpr int KP = D * 4 + 16;             // tile row pitch (bytes): rows 4 banks apart
    constexpr int K_BYTES = DF_KEYS * KP;
    constexpr int WAVE_BYTES = 2 * K_BYTES;    // K tile, V tile
    constexpr int CPR = D / 4;                 // 16-byte chunks per row
    constexpr int NLD = DF_KEYS * CPR / 64;    // 16-byte loads per lane per tile
    static_assert(DF_KEYS * CPR % 64 == 0, "a tile is a whole number of wavefront loads");
    constexpr int KC = D / 16;                 // 16-dim chunks of the contraction of K . Q^T
    constexpr int VW = (D % 64 == 0) ? 4 : 2;  // dims per V read
    constexpr int NBLK = D / (16 * VW);        // output blocks of 16 VW dims
    constexpr int COLS = DM_HEADS * CB;        // columns per workgroup
    constexpr int MERGE_BYTES = DEC_WAVES * COLS * (D + 2) * 4;
    constexpr int LDS_BYTES = DEC_WAVES * WAVE_BYTES > MERGE_BYTES ? DEC_WAVES * WAVE_BYTES : MERGE_BYTES;
    __shared__ __attribute__((aligned(16))) char smem[LDS_BYTES];

    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int j = lane & 15;  // column of this lane inside each block
    const int q4 = lane >> 4; // key group
    auto lds_base = (__attribute__((address_space(3))) char *)smem + wave * WAVE_BYTES;

    const int rows = p.Sq;  // columns are (query head, query row) pairs, see decode_mfma_kernel
    const int NC = p.G * rows;
    const int HB = (NC + COLS - 1) / COLS;
    int split, unit;
    if (!decode_unit_of_workgroup(p, p.B * p.Hkv * HB, &unit, &split)) return;
    const int hb = unit % HB;
    const int bg = unit / HB;
    const int g = bg % p.Hkv;
    const int b = bg / p.Hkv;
    const int c0 = hb * COLS;
    const int nh = min(COLS, NC - c0);
    int hj[CB], rj[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        const int cj = c0 + min(j + DM_HEADS * cb, nh - 1);
        hj[cb] = g * p.G + cj / rows, rj[cb] = cj % rows;
    }

    int kv_hi = p.Skv;
    if (p.kv_lens) kv_hi = min(kv_hi, max(p.kv_lens[b], 0));
    if (p.kv_lens && split * p.chunk >= kv_hi && split > 0) return;  // the combine pass skips it too
    int lo = split * p.chunk;
    int hi = min(lo + p.chunk, kv_hi);
    int lo_j[CB], hi_j[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        lo_j[cb] = lo, hi_j[cb] = hi;
        if (p.analytic && p.causal) hi_j[cb] = (int)min((int64_t)hi, p.q_pos_offset + 1 + rj[cb]);
        if (p.analytic && p.window > 0) lo_j[cb] = (int)max((int64_t)lo, p.q_pos_offset - p.window + 1 + rj[cb]);
    }
    if (p.analytic) {
        if (p.causal) hi = (int)min((int64_t)hi, p.q_pos_offset + rows);
        if (p.window > 0) lo = (int)max((int64_t)lo, p.q_pos_offset - p.window + 1);
    }

    const float *kbase = (const float *)p.k + b * p.ks[0] + g * p.ks[1];
    const float *vbase = (const float *)p.v + b * p.vs[0] + g * p.vs[1];
    const float *mrow[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        mrow[cb] = nullptr;
        if (p.mask_kind == FHIP_MASK_QK) mrow[cb] = (const float *)p.mask + rj[cb] * p.ms0;
        if (p.mask_kind == FHIP_MASK_BATCH_KEY) mrow[cb] = (const float *)p.mask + b * p.ms0;
    }
    const bool has_mask = p.mask_kind != FHIP_MASK_NONE;
    const float scale2 = p.scale * LOG2E;

    float4_t o[CB][NBLK][VW];
    float m[CB], l[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
#pragma unroll
        for (int nb = 0; nb < NBLK; nb++)
#pragma unroll
            for (int e = 0; e < VW; e++) o[cb][nb][e] = float4_t{0.f, 0.f, 0.f, 0.f};
        m[cb] = -INFINITY, l[cb] = 0.0f;
    }

    // one wavefront step = 16 consecutive keys; the four wavefronts interleave their steps.  Every lane always loads
    // (rows outside [lo, hi) are replaced by the nearest one inside; their scores are masked below).
    const int lo_al = lo - (lo % DF_KEYS);
    const int step = DEC_WAVES * DF_KEYS;
    float4_t kst[NLD], vst[NLD];
    auto load_tile = [&](int base) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < NLD; u++) {
            const int cid = lane + 64 * u;
            const int row = cid / CPR, col = cid % CPR;
            const int key = min(max(base + row, lo), hi - 1);
            kst[u] = __builtin_nontemporal_load((const float4_t *)(kbase + (int64_t)key * p.ks[2] + col * 4));
            vst[u] = __builtin_nontemporal_load((const float4_t *)(vbase + (int64_t)key * p.vs[2] + col * 4));
        }
    };
    auto store_tile = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < NLD; u++) {
            const int cid = lane + 64 * u;
            const int row = cid / CPR, col = cid % CPR;
            *DLDS_PTR(float4_t, row * KP + col * 16) = kst[u];
            *DLDS_PTR(float4_t, K_BYTES + row * KP + col * 16) = vst[u];
        }
    };

    int base = lo_al + wave * DF_KEYS;
    if (base < hi) load_tile(base);  // issued first so the Q fetch below overlaps it

    // Q^T operand: column j, dims 16 c + 4 q4 .. +4 (zero for the padding columns)
    float4_t qreg[CB][KC];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        const float *qp = (const float *)p.q + b * p.qs[0] + (int64_t)hj[cb] * p.qs[1] + (int64_t)rj[cb] * p.qs[2];
        const bool qvec = p.qs[3] == 1 && (((uintptr_t)qp) & 15) == 0;
#pragma unroll
        for (int c = 0; c < KC; c++) {
            float4_t v = {0.f, 0.f, 0.f, 0.f};
            if (j + DM_HEADS * cb < nh) {
                if (qvec) {
                    v = *(const float4_t *)(qp + 16 * c + 4 * q4);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = qp[(int64_t)(16 * c + 4 * q4 + e) * p.qs[3]];
                }
            }
            qreg[cb][c] = v;
        }
    }

    for (; base < hi; base += step) {
        wave_lds_sync();  // the previous step's LDS reads precede these writes
        store_tile();
        wave_lds_sync();
        load_tile(base + step);  // in flight during the math below (beyond the end: a row read again)

        // ---- S^T[key][col] = K . Q^T : every K operand read serves all column blocks ----------------------
        float4_t s[CB];
#pragma unroll
        for (int cb = 0; cb < CB; cb++) s[cb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KC; c++) {
            const float4_t a = *DLDS_PTR(float4_t, j * KP + (16 * c + 4 * q4) * 4);
#pragma unroll
            for (int cb = 0; cb < CB; cb++)
#pragma unroll
                for (int i = 0; i < 4; i++) s[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], qreg[cb][c][i], s[cb], 0, 0, 0);
        }
        float pe[CB][4];
#pragma unroll
        for (int cb = 0; cb < CB; cb++) {
            // element r is key base + 4 q4 + r for column j of block cb
            float sv[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int key = base + 4 * q4 + r;
                const bool visible = key >= lo_j[cb] && key < hi_j[cb];
                float x = s[cb][r] * scale2;
                if (has_mask && visible) x += mrow[cb][(int64_t)key * p.ms1] * LOG2E;
                sv[r] = visible ? x : -INFINITY;
            }
            float mx = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
            mx = quad_rows_max(mx);
            const float m_new = fmaxf(m[cb], mx);
            const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
            const float corr = __builtin_amdgcn_exp2f(m[cb] - m_safe);
            m[cb] = m_new;
            float psum = 0.0f;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                pe[cb][r] = __builtin_amdgcn_exp2f(sv[r] - m_safe);
                psum += pe[cb][r];
            }
            l[cb] = l[cb] * corr + psum;
#pragma unroll
            for (int nb = 0; nb < NBLK; nb++)
#pragma unroll
                for (int e = 0; e < VW; e++)
#pragma unroll
                    for (int r = 0; r < 4; r++) o[cb][nb][e][r] *= corr;
        }

        // ---- O^T[dim][col] += V^T . P^T : step ks contracts the keys 4 q4 + ks ----------------------------
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
#pragma unroll
            for (int nb = 0; nb < NBLK; nb++) {
                const int voff = K_BYTES + (4 * q4 + ks) * KP + (16 * VW * nb + VW * j) * 4;
                if constexpr (VW == 4) {
                    const float4_t a = *DLDS_PTR(float4_t, voff);
#pragma unroll
                    for (int cb = 0; cb < CB; cb++)
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            o[cb][nb][e] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], pe[cb][ks], o[cb][nb][e], 0, 0, 0);
                } else {
                    typedef float float2v_t __attribute__((ext_vector_type(2)));
                    const float2v_t a = *DLDS_PTR(float2v_t, voff);
#pragma unroll
                    for (int cb = 0; cb < CB; cb++)
#pragma unroll
                        for (int e = 0; e < 2; e++)
                            o[cb][nb][e] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], pe[cb][ks], o[cb][nb][e], 0, 0, 0);
                }
            }
        }
    }

    // ---- merge: key groups -> wavefront -> workgroup ------------------------------------------------
    __syncthreads();  // every wavefront is done with its K/V tile; the LDS is reused for the merge
    float *macc = (float *)smem;  // [wave][column][D + 2]
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        const float l_col = quad_rows_sum(l[cb]);
        if (j + DM_HEADS * cb < nh) {
            float *dst = macc + ((wave * COLS + j + DM_HEADS * cb) * (D + 2));
            // element (nb, e, r) of this lane is dim 16 VW nb + VW (4 q4 + r) + e
#pragma unroll
            for (int nb = 0; nb < NBLK; nb++)
#pragma unroll
                for (int e = 0; e < VW; e++)
#pragma unroll
                    for (int r = 0; r < 4; r++) dst[16 * VW * nb + VW * (4 * q4 + r) + e] = o[cb][nb][e][r];
            if (q4 == 0) {
                dst[D] = m[cb];
                dst[D + 1] = l_col;
            }
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < nh * D; idx += 64 * DEC_WAVES) {
        const int hh = idx / D, d = idx % D;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; w++) M = fmaxf(M, macc[(w * COLS + hh) * (D + 2) + D]);
        const float Ms = (M == -INFINITY) ? 0.0f : M;
        float L = 0.0f, A = 0.0f;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; w++) {
            const float *src = macc + (w * COLS + hh) * (D + 2);
            const float wgt = __builtin_amdgcn_exp2f(src[D] - Ms);
            L += wgt * src[D + 1];
            A += wgt * src[d];
        }
        const int h = g * p.G + (c0 + hh) / rows, qr = (c0 + hh) % rows;
        if (p.nsplit == 1) {
            ((float *)p.out)[b * p.os[0] + h * p.os[1] + qr * p.os[2] + d * p.os[3]] = A / L;  // no visible key: 0/0 = NaN
        } else {
            float *ws = p.dec_fused
                            ? fused_partial_row(p, unit, split, hh, D)
                            : (float *)p.partials + ((((int64_t)b * p.H + h) * rows + qr) * p.nsplit + split) * (D + 2);
            ws[d] = A;
            if (d == 0) {
                ws[D] = M;
                ws[D + 1] = L;
            }
        }
    }
    if (p.dec_fused && p.nsplit > 1) fused_merge_tail<float, 64 * DEC_WAVES>(p, unit, nh, D, b, g, c0, rows);
}

// ---- pass 2 -------------------------------------------------------------------------------------
// One 64-lane wavefront per (batch, head); up to U partials are fetched in one round of loads (a round costs
// one memory latency, so calls with many splits take the wide form).

template <typename T, int U>
__global__ __launch_bounds__(64) void decode_combine_kernel(AttnParams p) {
    const int qr = blockIdx.x % p.Sq, bh = blockIdx.x / p.Sq;  // one workgroup per (batch, head, query row)
    const int h = bh % p.H, b = bh / p.H;
    const int D = p.D;
    int ns = p.nsplit;
    if (p.kv_lens) {
        const int len = min(p.Skv, max(p.kv_lens[b], 0));
        ns = max(1, min(ns, (len + p.chunk - 1) / p.chunk));  // split 0 is always written
    }
    const float *ws = (const float *)p.partials + (int64_t)blockIdx.x * p.nsplit * (D + 2);
    const int64_t ob = b * p.os[0] + h * p.os[1] + qr * p.os[2];
    // 128 dims per round (one round up to head_dim 128, two at 256)
    for (int dbase = 0; dbase < D; dbase += 128) {
        const int d0 = dbase + threadIdx.x, d1 = dbase + threadIdx.x + 64;
        float M = -INFINITY, L = 0.0f, A0 = 0.0f, A1 = 0.0f;
        for (int s0 = 0; s0 < ns; s0 += U) {
            float ms[U], ls[U], a0[U], a1[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const bool ok = s0 + u < ns;
                const float *src = ws + (int64_t)(ok ? s0 + u : s0) * (D + 2);
                ms[u] = ok ? src[D] : -INFINITY;
                ls[u] = ok ? src[D + 1] : 0.0f;
                a0[u] = (ok && d0 < D) ? src[d0] : 0.0f;
                a1[u] = (ok && d1 < D) ? src[d1] : 0.0f;
            }
            float Mn = M;
#pragma unroll
            for (int u = 0; u < U; u++) Mn = fmaxf(Mn, ms[u]);
            const float Ms = (Mn == -INFINITY) ? 0.0f : Mn;
            const float c = __builtin_amdgcn_exp2f(M - Ms);
            L *= c;
            A0 *= c;
            A1 *= c;
#pragma unroll
            for (int u = 0; u < U; u++) {
                const float w = __builtin_amdgcn_exp2f(ms[u] - Ms);
                L += w * ls[u];
                A0 += w * a0[u];
                A1 += w * a1[u];
            }
            M = Mn;
        }
        if (d0 < D) {
            const float val = A0 / L;
            if (p.out_f32) ((float *)p.out)[ob + d0 * p.os[3]] = val;
            else ((T *)p.out)[ob + d0 * p.os[3]] = from_float<T>(val);
        }
        if (d1 < D) {
            const float val = A1 / L;
            if (p.out_f32) ((float *)p.out)[ob + d1 * p.os[3]] = val;
            else ((T *)p.out)[ob + d1 * p.os[3]] = from_float<T>(val);
        }
    }
}

// Few (batch, head) rows with many splits (batch 1 on a long cache): one wavefront per row leaves the chip empty
// and issues every load of a row from 64 lanes.  Here four wavefronts share a row, each merges a quarter of the
// splits (U in flight per lane), and the first folds the four states through LDS.
template <typename T, int U>
__global__ __launch_bounds__(256) void decode_combine4_kernel(AttnParams p) {
    __shared__ float part[4][2 + 128];
    const int qr = blockIdx.x % p.Sq, bh = blockIdx.x / p.Sq;  // one workgroup per (batch, head, query row)
    const int h = bh % p.H, b = bh / p.H;
    const int D = p.D;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int ns = p.nsplit;
    if (p.kv_lens) {
        const int len = min(p.Skv, max(p.kv_lens[b], 0));
        ns = max(1, min(ns, (len + p.chunk - 1) / p.chunk));  // split 0 is always written
    }
    const float *ws = (const float *)p.partials + (int64_t)blockIdx.x * p.nsplit * (D + 2);
    const int64_t ob = b * p.os[0] + h * p.os[1] + qr * p.os[2];
    const int per = (ns + 3) / 4, s_lo = wave * per, s_hi = min(ns, s_lo + per);
    for (int dbase = 0; dbase < D; dbase += 128) {
        const int d0 = dbase + lane, d1 = dbase + lane + 64;
        float M = -INFINITY, L = 0.0f, A0 = 0.0f, A1 = 0.0f;
        for (int s0 = s_lo; s0 < s_hi; s0 += U) {
            float ms[U], ls[U], a0[U], a1[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const bool ok = s0 + u < s_hi;
                const float *src = ws + (int64_t)(ok ? s0 + u : s0) * (D + 2);
                ms[u] = ok ? src[D] : -INFINITY;
                ls[u] = ok ? src[D + 1] : 0.0f;
                a0[u] = (ok && d0 < D) ? src[d0] : 0.0f;
                a1[u] = (ok && d1 < D) ? src[d1] : 0.0f;
            }
            float Mn = M;
#pragma unroll
            for (int u = 0; u < U; u++) Mn = fmaxf(Mn, ms[u]);
            const float Ms = (Mn == -INFINITY) ? 0.0f : Mn;
            const float c = __builtin_amdgcn_exp2f(M - Ms);
            L *= c;
            A0 *= c;
            A1 *= c;
#pragma unroll
            for (int u = 0; u < U; u++) {
                const float w = __builtin_amdgcn_exp2f(ms[u] - Ms);
                L += w * ls[u];
                A0 += w * a0[u];
                A1 += w * a1[u];
            }
            M = Mn;
        }
        if (dbase > 0) __syncthreads();  // the previous round's states have been read
        part[wave][2 + lane] = A0;
        part[wave][2 + 64 + lane] = A1;
        if (lane == 0) {
            part[wave][0] = M;
            part[wave][1] = L;
        }
        __syncthreads();
        if (wave == 0) {
            float Mn = -INFINITY;
#pragma unroll
            for (int w = 0; w < 4; w++) Mn = fmaxf(Mn, part[w][0]);
            const float Ms = (Mn == -INFINITY) ? 0.0f : Mn;
            float Lt = 0.0f, B0 = 0.0f, B1 = 0.0f;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const float c = __builtin_amdgcn_exp2f(part[w][0] - Ms);
                Lt += c * part[w][1];
                B0 += c * part[w][2 + lane];
                B1 += c * part[w][2 + 64 + lane];
            }
            if (d0 < D) {
                const float val = B0 / Lt;  // no visible key: 0/0 = NaN like the reference
                if (p.out_f32) ((float *)p.out)[ob + d0 * p.os[3]] = val;
                else ((T *)p.out)[ob + d0 * p.os[3]] = from_float<T>(val);
            }
            if (d1 < D) {
                const float val = B1 / Lt;
                if (p.out_f32) ((float *)p.out)[ob + d1 * p.os[3]] = val;
                else ((T *)p.out)[ob + d1 * p.os[3]] = from_float<T>(val);
            }
        }
    }
}

template <typename T>
static void launch_combine(const AttnParams &p, hipStream_t stream) {
    const dim3 grid((unsigned)(p.B * p.H * p.Sq)), block(64);
    const int cus = p.cus > 0 ? p.cus : 256;
    if (p.nsplit <= 8) hipLaunchKernelGGL((decode_combine_kernel<T, 8>), grid, block, 0, stream, p);
    else if ((long)p.B * p.H * p.Sq > 2L * cus) hipLaunchKernelGGL((decode_combine_kernel<T, 32>), grid, block, 0, stream, p);
    else if (p.nsplit <= 32) hipLaunchKernelGGL((decode_combine4_kernel<T, 8>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((decode_combine4_kernel<T, 16>), grid, dim3(256), 0, stream, p);
}

template <typename T, int LPK>
static void launch_vec(const AttnParams &p, dim3 grid, hipStream_t stream, int gt) {
    dim3 block(64 * DEC_WAVES);
    switch (gt) {
        case 1: FHIP_LAUNCH_MAIN((decode_vec_kernel<T, LPK, 1>), grid, block, stream, p, p); break;
        case 2: FHIP_LAUNCH_MAIN((decode_vec_kernel<T, LPK, 2>), grid, block, stream, p, p); break;
        case 4: FHIP_LAUNCH_MAIN((decode_vec_kernel<T, LPK, 4>), grid, block, stream, p, p); break;
        default: FHIP_LAUNCH_MAIN((decode_vec_kernel<T, LPK, 8>), grid, block, stream, p, p); break;
    }
}

// the matrix-core variants by head_dim; above 128 only the form with four wavefronts and one column block exists
template <typename T, int WAVES, int CB>
static void launch_mfma_16(const AttnParams &p, dim3 grid, hipStream_t stream) {
    const dim3 block(64 * WAVES);
    switch (p.D) {
        case 32: FHIP_LAUNCH_MAIN((decode_mfma_kernel<T, 32, WAVES, CB>), grid, block, stream, p, p); return;
        case 64: FHIP_LAUNCH_MAIN((decode_mfma_kernel<T, 64, WAVES, CB>), grid, block, stream, p, p); return;
        case 96: FHIP_LAUNCH_MAIN((decode_mfma_kernel<T, 96, WAVES, CB>), grid, block, stream, p, p); return;
        case 128: FHIP_LAUNCH_MAIN((decode_mfma_kernel<T, 128, WAVES, CB>), grid, block, stream, p, p); return;
        default: break;
    }
    if constexpr (WAVES == DEC_WAVES && CB == 1) {
        switch (p.D) {
            case 160: FHIP_LAUNCH_MAIN((decode_mfma_kernel<T, 160, WAVES, 1>), grid, block, stream, p, p); return;
            case 192: FHIP_LAUNCH_MAIN((decode_mfma_kernel<T, 192, WAVES, 1>), grid, block, stream, p, p); return;
            case 224: FHIP_LAUNCH_MAIN((decode_mfma_kernel<T, 224, WAVES, 1>), grid, block, stream, p, p); return;
            default: FHIP_LAUNCH_MAIN((decode_mfma_kernel<T, 256, WAVES, 1>), grid, block, stream, p, p); return;
        }
    }
}
template <int CB>
static void launch_mfma_f32(const AttnParams &p, dim3 grid, hipStream_t stream) {
    const dim3 block(64 * DEC_WAVES);
    switch (p.D) {
        case 32: FHIP_LAUNCH_MAIN((decode_mfma_f32_kernel<32, CB>), grid, block, stream, p, p); return;
        case 64: FHIP_LAUNCH_MAIN((decode_mfma_f32_kernel<64, CB>), grid, block, stream, p, p); return;
        case 96: FHIP_LAUNCH_MAIN((decode_mfma_f32_kernel<96, CB>), grid, block, stream, p, p); return;
        case 128: FHIP_LAUNCH_MAIN((decode_mfma_f32_kernel<128, CB>), grid, block, stream, p, p); return;
        default: break;
    }
    if (p.D == 160) FHIP_LAUNCH_MAIN((decode_mfma_f32_kernel<160, CB>), grid, block, stream, p, p);
    else if (p.D == 192) FHIP_LAUNCH_MAIN((decode_mfma_f32_kernel<192, CB>), grid, block, stream, p, p);
    if constexpr (CB == 1) {
        if (p.D == 224) FHIP_LAUNCH_MAIN((decode_mfma_f32_kernel<224, 1>), grid, block, stream, p, p);
        else if (p.D == 256) FHIP_LAUNCH_MAIN((decode_mfma_f32_kernel<256, 1>), grid, block, stream, p, p);
    }
}

template <typename T>
static int launch_decode_t(const AttnParams &p, hipStream_t stream) {
    constexpr bool F32 = sizeof(T) == 4;
    const int gt = decode_gt(p.G * p.Sq, p.D, F32);  // columns: (query head, query row) pairs of a KV head
    const int hb = (p.G * p.Sq + gt - 1) / gt;
    const long gy = (long)p.B * p.Hkv * hb;
    if (gy > 65535 || p.nsplit > 0x7fffffff) {
        set_error("decode: batch * kv_heads * head_blocks = %ld exceeds the grid limit 65535", gy);
        return FHIP_ERR_UNSUPPORTED;
    }
    dim3 grid((unsigned)p.nsplit, (unsigned)gy);
    if (p.dec_fused) grid = dim3((unsigned)((gy + 7) / 8 * 8 * p.nsplit));  // see the kernel's unit numbering
    if constexpr (F32) {
        if (decode_use_mfma(p.D, true, p.G * p.Sq)) {
            if (gt == 32) launch_mfma_f32<2>(p, grid, stream);
            else launch_mfma_f32<1>(p, grid, stream);
            FHIP_HIP_CHECK(hipGetLastError());
            FHIP_MARK_MAIN_DONE(p, stream);
            if (p.nsplit > 1 && !p.dec_fused) {
                launch_combine<T>(p, stream);
                FHIP_HIP_CHECK(hipGetLastError());
            }
            return FHIP_OK;
        }
    }
    if constexpr (!F32) {
        if (decode_use_mfma(p.D, false, p.G * p.Sq)) {
            if (p.dec_waves == 8) {
                if (gt == 32) launch_mfma_16<T, 8, 2>(p, grid, stream);
                else launch_mfma_16<T, 8, 1>(p, grid, stream);
            } else {
                if (gt == 32) launch_mfma_16<T, DEC_WAVES, 2>(p, grid, stream);
                else launch_mfma_16<T, DEC_WAVES, 1>(p, grid, stream);
            }
            FHIP_HIP_CHECK(hipGetLastError());
            FHIP_MARK_MAIN_DONE(p, stream);
            if (p.nsplit > 1 && !p.dec_fused) {
                launch_combine<T>(p, stream);
                FHIP_HIP_CHECK(hipGetLastError());
            }
            return FHIP_OK;
        }
    }
    if (p.D <= 32) {
        launch_vec<T, 4>(p, grid, stream, gt);
    } else if (p.D <= 64) {
        launch_vec<T, 8>(p, grid, stream, gt);
    } else if (p.D <= 128) {
        launch_vec<T, 16>(p, grid, stream, gt);
    } else {
        launch_vec<T, 32>(p, grid, stream, gt);
    }
    FHIP_HIP_CHECK(hipGetLastError());
    FHIP_MARK_MAIN_DONE(p, stream);
    if (p.nsplit > 1) {
        launch_combine<T>(p, stream);
        FHIP_HIP_CHECK(hipGetLastError());
    }
    return FHIP_OK;
}

int launch_decode(const AttnParams &p, fhip_dtype dtype, hipStream_t stream) {
    if (dtype == FHIP_F16) return launch_decode_t<half_t>(p, stream);
    if (dtype == FHIP_BF16) return launch_decode_t<bf16_t>(p, stream);
    return launch_decode_t<float>(p, stream);
}

}  // namespace fhip
