// Rotary position embedding, fused with the type conversion and the write into its destination
// (a query tensor for the attention call, or the new rows of the KV cache).
//
// Semantics: fusor-ml/fusor/src/composite/rope.rs:46-137 in f32, one rounding per operation as the
// reference's CPU path has (mul, mul, add are separate tensor ops there):
//   normal (rope / rope_normal_fused):       y[i]        = x[i] * cos[p][i]        + (-x[i + D/2]) * sin[p][i]
//                                            y[i + D/2]  = x[i + D/2] * cos[p][i]  +   x[i]        * sin[p][i]
//   interleaved (rope_interleaved / rope_fused): y[2i]   = x[2i] * cos[p][i] - x[2i+1] * sin[p][i]
//                                            y[2i+1]     = x[2i] * sin[p][i] + x[2i+1] * cos[p][i]
// with p = start_pos + row (RopeCache::forward, rope.rs:232-265) and cos/sin the [positions, D/2]
// f32 tables of fusor::RopeCache.  16-bit inputs are widened to f32 first and the result is rounded
// to nearest even, which is what kalosm-llama's cast -> rope -> cast does
// (models/kalosm-llama/src/raw/rope.rs:103-111).
//
// Optionally the row is RMS-normalised first (the q / k norm of Qwen3- and Gemma3-style blocks,
// models/kalosm-llama/src/raw/attention_layer.rs:229-235,251-257 -> RmsNorm::forward_generic_4d,
// fusor-ml/fusor/src/layers/rms_norm.rs:122-133 -> rms_norm_fused_cpu_impl,
// fusor-ml/fusor/src/composite/normalization.rs:351-407), again one rounding per operation and in the
// reference's order:
//   ss = fold(+, 0, x[i] * x[i]) left to right;  rms = sqrt(ss / D + eps);  n[i] = (x[i] / rms) * w[i] (+ bias[i])
// and n is rounded to the tensor's element type before the rotation, because the reference's norm returns a
// tensor of that type.
#include "common.h"
#include "device_utils.h"

namespace fhip {

__device__ __forceinline__ float load_as_f32(const void *p, int64_t idx, int dtype) {
    if (dtype == FHIP_F32) return ((const float *)p)[idx];
    if (dtype == FHIP_F16) return (float)((const half_t *)p)[idx];
    return to_float(((const bf16_t *)p)[idx]);
}
__device__ __forceinline__ void store_from_f32(void *p, int64_t idx, int dtype, float v) {
    if (dtype == FHIP_F32) ((float *)p)[idx] = v;
    else if (dtype == FHIP_F16) ((half_t *)p)[idx] = (half_t)v;
    else ((bf16_t *)p)[idx] = from_float<bf16_t>(v);
}

__device__ __forceinline__ float round_through(float v, int dtype) {
    if (dtype == FHIP_F16) return (float)(half_t)v;
    if (dtype == FHIP_BF16) return to_float(from_float<bf16_t>(v));
    return v;
}

// ---- 16 bytes (f32) / 8 bytes (16-bit) at a time -------------------------------------------------
// The fast forms below need rows whose elements are consecutive and whose starts are aligned to four
// elements on both sides, and a head_dim that is a multiple of 8 (fill_row_job checks; `vec`).
typedef uint32_t uint2r_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float4_t load4_as_f32(const void *p, int64_t idx, int dtype) {
    if (dtype == FHIP_F32) return *(const float4_t *)((const float *)p + idx);
    const uint2r_t raw = *(const uint2r_t *)((const uint16_t *)p + idx);
    float4_t v;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const uint16_t bits = (uint16_t)(raw[e >> 1] >> (16 * (e & 1)));
        v[e] = dtype == FHIP_F16 ? (float)__builtin_bit_cast(half_t, bits) : __uint_as_float((uint32_t)bits << 16);
    }
    return v;
}
__device__ __forceinline__ void store4_from_f32(void *p, int64_t idx, int dtype, float4_t v) {
    if (dtype == FHIP_F32) {
        *(float4_t *)((float *)p + idx) = v;
        return;
    }
    uint32_t bits[4];
#pragma unroll
    for (int e = 0; e < 4; e++)
        bits[e] = dtype == FHIP_F16 ? (uint32_t)__builtin_bit_cast(uint16_t, (half_t)v[e]) : (uint32_t)from_float<bf16_t>(v[e]).bits;
    *(uint2r_t *)((uint16_t *)p + idx) = uint2r_t{bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16)};
}

// element offsets of row t (a flat index over [B, heads, rows]) in the source and the destination, and its position
__device__ __forceinline__ void row_bases(const RopeRows &a, int64_t t, int64_t *sb, int64_t *db, uint32_t *r) {
    *r = (uint32_t)(t % a.shape[2]);
    t /= a.shape[2];
    const int64_t h = t % a.shape[1], b = t / a.shape[1];
    *sb = b * a.ss[0] + h * a.ss[1] + *r * a.ss[2];
    *db = b * a.ds[0] + h * a.ds[1] + *r * a.ds[2];
}

// Rotation / conversion without the norm, four pairs (or four elements) per lane and step: every load and store is
// 16 bytes of f32 or 8 bytes of a 16-bit type, consecutive lanes take consecutive pieces of a row.
__device__ __forceinline__ void rope_rows_vec_body(const RopeRows &a) {
    const uint32_t D = a.shape[3], half = D / 2;
    const uint32_t upr = a.mode == 2 ? D / 4 : half / 4;  // steps per row
    const int64_t total = (int64_t)a.shape[0] * a.shape[1] * a.shape[2] * upr;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const uint32_t j = (uint32_t)(idx % upr);
        int64_t sb, db;
        uint32_t r;
        row_bases(a, idx / upr, &sb, &db, &r);
        if (a.mode == 2) {
            store4_from_f32(a.dst, db + 4 * j, a.dst_dtype, load4_as_f32(a.src, sb + 4 * j, a.src_dtype));
            continue;
        }
        const float4_t c = *(const float4_t *)(a.cos + (a.pos0 + r) * half + 4 * j);
        const float4_t s = *(const float4_t *)(a.sin + (a.pos0 + r) * half + 4 * j);
        float4_t ya, yb;
        if (a.mode == 0) {  // pairs (4j + e, half + 4j + e)
            const float4_t x0 = load4_as_f32(a.src, sb + 4 * j, a.src_dtype);
            const float4_t x1 = load4_as_f32(a.src, sb + half + 4 * j, a.src_dtype);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                ya[e] = __fsub_rn(__fmul_rn(x0[e], c[e]), __fmul_rn(x1[e], s[e]));
                yb[e] = __fadd_rn(__fmul_rn(x1[e], c[e]), __fmul_rn(x0[e], s[e]));
            }
            store4_from_f32(a.dst, db + 4 * j, a.dst_dtype, ya);
            store4_from_f32(a.dst, db + half + 4 * j, a.dst_dtype, yb);
        } else {  // pairs (8j + 2e, 8j + 2e + 1)
            const float4_t xa = load4_as_f32(a.src, sb + 8 * j, a.src_dtype);
            const float4_t xb = load4_as_f32(a.src, sb + 8 * j + 4, a.src_dtype);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float x0 = e < 2 ? xa[2 * e] : xb[2 * e - 4], x1 = e < 2 ? xa[2 * e + 1] : xb[2 * e - 3];
                const float y0 = __fsub_rn(__fmul_rn(x0, c[e]), __fmul_rn(x1, s[e]));
                const float y1 = __fadd_rn(__fmul_rn(x0, s[e]), __fmul_rn(x1, c[e]));
                if (e < 2) ya[2 * e] = y0, ya[2 * e + 1] = y1;
                else yb[2 * e - 4] = y0, yb[2 * e - 3] = y1;
            }
            store4_from_f32(a.dst, db + 8 * j, a.dst_dtype, ya);
            store4_from_f32(a.dst, db + 8 * j + 4, a.dst_dtype, yb);
        }
    }
}

// The normalised variant on whole row blocks.  The sum of squares of a row is one lane's left-to-right fold (the
// order fixes the rounding), so a wavefront parks a block of rows in its own LDS tile with wide, consecutive loads
// (pitch head_dim + 1 floats: the lanes then fold their rows without bank conflicts), every lane that has a row
// folds it, all lanes normalise and rotate the pairs in place, and the tile leaves with wide stores.  The rows of a
// block are all read before any is written, so the destination may be the source.
constexpr int NORM_TILE_FLOATS = 2112;  // per wavefront: 16 rows of head_dim 128, 32 of 64, 8 of 256
struct NormWaveLds {
    float tile[NORM_TILE_FLOATS];
    int64_t sb[64], db[64];  // element offsets of the block's rows in the source and the destination
    uint32_t pos[64];        // their positions (rows of the cos / sin tables, before pos0)
    float rms[64];
};
// FEW: the block's rows divided by FEW (1 or 4: down to 8 / 4 / 2 rows at head_dim 64 / 128 / 256), for inputs whose
// blocks of the full size would leave most SIMDs with one wavefront or none: a block's stages (fetch, fold, normalise,
// store) run one after the other, so a prompt of a few hundred rows is bound by one block's latencies, not by the
// arithmetic.
template <int D, int FEW>
__device__ __forceinline__ void norm_rope_rows_vec_body(const RopeRows &a, NormWaveLds *w) {
    constexpr int HALF = D / 2, CPR = D / 4, P = D + 1;
    static_assert(CPR <= 64 && 64 % CPR == 0 && D % 64 == 0, "head_dim 64, 128 or 256");
    // A wavefront step moves RS rows: lane -> (row SUB of the step, 16-byte piece C4 of the row).  The pairs of a row
    // likewise: lane -> (row psub of the step, pair pi), PP steps per row beyond 64 pairs.  A block is LSTEPS load
    // steps = PSTEPS pair steps, all requested before the first is parked.
    constexpr int RS = 64 / CPR;
    constexpr int PRS = HALF <= 64 ? 64 / HALF : 1, PP = HALF <= 64 ? 1 : HALF / 64;
    constexpr int RPW = (D == 64 ? 32 : D == 128 ? 16 : 8) / FEW;  // rows per block
    constexpr int LSTEPS = RPW / RS, PSTEPS = RPW * PP / PRS;
    static_assert(RPW * P <= NORM_TILE_FLOATS, "tile");
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwave = blockDim.x >> 6;
    float *tile = w->tile;
    const int sub = lane / CPR, c4 = lane % CPR;
    const int psub = HALF <= 64 ? lane / HALF : 0, pi = HALF <= 64 ? lane % HALF : lane;
    const int64_t rows = (int64_t)a.shape[0] * a.shape[1] * a.shape[2];
    const int64_t nblk = (rows + RPW - 1) / RPW;
    // weights (and bias) of this lane's pairs: the same for every row
    float w0[PP], w1[PP], b0[PP], b1[PP];
#pragma unroll
    for (int k = 0; k < PP; k++) {
        const int i = pi + 64 * k;
        const int d0 = a.mode == 0 ? i : 2 * i, d1 = a.mode == 0 ? i + HALF : 2 * i + 1;
        w0[k] = load_as_f32(a.norm_w, d0, a.norm_dtype), w1[k] = load_as_f32(a.norm_w, d1, a.norm_dtype);
        b0[k] = a.norm_b ? load_as_f32(a.norm_b, d0, a.norm_dtype) : 0.0f;
        b1[k] = a.norm_b ? load_as_f32(a.norm_b, d1, a.norm_dtype) : 0.0f;
    }
    const bool small = rows < (int64_t)0x7fffffff;
    for (int64_t blk = (int64_t)blockIdx.x * nwave + wave; blk < nblk; blk += (int64_t)gridDim.x * nwave) {
        const int64_t row0 = blk * RPW;
        const int nrow = (int)min((int64_t)RPW, rows - row0);
        if (lane < nrow) {
            int64_t sb, db;
            uint32_t r;
            if (small) {  // 32-bit divisions
                uint32_t t = (uint32_t)(row0 + lane);
                r = t % a.shape[2];
                t /= a.shape[2];
                const uint32_t h = t % a.shape[1], b = t / a.shape[1];
                sb = b * a.ss[0] + h * a.ss[1] + r * a.ss[2];
                db = b * a.ds[0] + h * a.ds[1] + r * a.ds[2];
            } else {
                row_bases(a, row0 + lane, &sb, &db, &r);
            }
            w->sb[lane] = sb, w->db[lane] = db, w->pos[lane] = r;
        }
        wave_lds_sync();
        float4_t x[LSTEPS];
#pragma unroll
        for (int u = 0; u < LSTEPS; u++) {
            const int lr = u * RS + sub;
            if (lr < nrow) x[u] = load4_as_f32(a.src, w->sb[lr] + 4 * c4, a.src_dtype);
        }
        float tc[PSTEPS], ts[PSTEPS];
#pragma unroll
        for (int q = 0; q < PSTEPS; q++) {
            const int lr = PP == 1 ? q * PRS + psub : q / PP;
            const int i = pi + 64 * (q % PP);
            tc[q] = 1.0f, ts[q] = 0.0f;
            if (a.mode != 2 && lr < nrow) {
                const int64_t ti = (a.pos0 + w->pos[lr]) * HALF + i;
                tc[q] = a.cos[ti], ts[q] = a.sin[ti];
            }
        }
#pragma unroll
        for (int u = 0; u < LSTEPS; u++) {
            const int lr = u * RS + sub;
            if (lr < nrow) {
#pragma unroll
                for (int e = 0; e < 4; e++) tile[lr * P + 4 * c4 + e] = x[u][e];
            }
        }
        wave_lds_sync();
        if (lane < nrow) {
            float ss = 0.0f;
#pragma unroll 2
            for (int i = 0; i < D; i += 8) {  // eight values requested before the dependent chain consumes them
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; e++) v[e] = tile[lane * P + i + e];
#pragma unroll
                for (int e = 0; e < 8; e++) ss = __fadd_rn(ss, __fmul_rn(v[e], v[e]));
            }
            // sqrtf is the correctly rounded root (the __fsqrt_rn intrinsic is the 1-ulp hardware approximation here)
            w->rms[lane] = sqrtf(__fadd_rn(__fdiv_rn(ss, (float)D), a.eps));
        }
        wave_lds_sync();
        // a pair: normalise both elements, round to the tensor's type as the reference's norm does, rotate
#pragma unroll
        for (int q = 0; q < PSTEPS; q++) {
            const int lr = PP == 1 ? q * PRS + psub : q / PP;
            const int k = q % PP, i = pi + 64 * k;
            if (lr >= nrow) continue;
            const int d0 = a.mode == 0 ? i : 2 * i, d1 = a.mode == 0 ? i + HALF : 2 * i + 1;
            const float rms = w->rms[lr];
            float x0 = __fmul_rn(__fdiv_rn(tile[lr * P + d0], rms), w0[k]);
            float x1 = __fmul_rn(__fdiv_rn(tile[lr * P + d1], rms), w1[k]);
            if (a.norm_b) {
                x0 = __fadd_rn(x0, b0[k]);
                x1 = __fadd_rn(x1, b1[k]);
            }
            x0 = round_through(x0, a.src_dtype);
            x1 = round_through(x1, a.src_dtype);
            float y0 = x0, y1 = x1;
            if (a.mode != 2) {
                y0 = __fsub_rn(__fmul_rn(x0, tc[q]), __fmul_rn(x1, ts[q]));
                y1 = a.mode == 0 ? __fadd_rn(__fmul_rn(x1, tc[q]), __fmul_rn(x0, ts[q]))
                                 : __fadd_rn(__fmul_rn(x0, ts[q]), __fmul_rn(x1, tc[q]));
            }
            tile[lr * P + d0] = y0;
            tile[lr * P + d1] = y1;
        }
        wave_lds_sync();
#pragma unroll
        for (int u = 0; u < LSTEPS; u++) {
            const int lr = u * RS + sub;
            if (lr < nrow) {
                float4_t y;
#pragma unroll
                for (int e = 0; e < 4; e++) y[e] = tile[lr * P + 4 * c4 + e];
                store4_from_f32(a.dst, w->db[lr] + 4 * c4, a.dst_dtype, y);
            }
        }
        wave_lds_sync();  // the tile and the row tables are rewritten by the next block
    }
}
__device__ __forceinline__ void norm_rope_rows_vec_any(const RopeRows &a, NormWaveLds *w) {
    if (a.few == 4) {
        if (a.shape[3] == 128) norm_rope_rows_vec_body<128, 4>(a, w);
        else if (a.shape[3] == 256) norm_rope_rows_vec_body<256, 4>(a, w);
        else norm_rope_rows_vec_body<64, 4>(a, w);
        return;
    }
    if (a.shape[3] == 128) norm_rope_rows_vec_body<128, 1>(a, w);
    else if (a.shape[3] == 256) norm_rope_rows_vec_body<256, 1>(a, w);
    else norm_rope_rows_vec_body<64, 1>(a, w);
}

// The general form of the normalised variant (any strides): a workgroup takes groups of rows; one lane per row folds the squares in the
// reference's left-to-right order (the order fixes the rounding, so the sum is not split over lanes), the
// row's rms goes through LDS, then one lane per pair normalises and rotates as below.
constexpr int NORM_ROPE_MAX_ROWS = 256;
__device__ __forceinline__ void norm_rope_rows_body(const RopeRows &a, float *rms_of) {
    const uint32_t D = a.shape[3], half = D / 2;
    const int64_t rows = (int64_t)a.shape[0] * a.shape[1] * a.shape[2];
    const int rpb = half >= 256 ? 1 : 256 / half;  // rows per group
    const int tid = threadIdx.x;
    for (int64_t row0 = (int64_t)blockIdx.x * rpb; row0 < rows; row0 += (int64_t)gridDim.x * rpb) {
        const int nrow = (int)min((int64_t)rpb, rows - row0);
        if (tid < nrow) {
            int64_t t = row0 + tid;
            const uint32_t r = (uint32_t)(t % a.shape[2]);
            t /= a.shape[2];
            const int64_t sb = (t / a.shape[1]) * a.ss[0] + (t % a.shape[1]) * a.ss[1] + r * a.ss[2];
            float ss = 0.0f;
            for (uint32_t i = 0; i < D; i++) {
                const float x = load_as_f32(a.src, sb + i * a.ss[3], a.src_dtype);
                ss = __fadd_rn(ss, __fmul_rn(x, x));
            }
            // sqrtf is the correctly rounded root (the __fsqrt_rn intrinsic is the 1-ulp hardware approximation here)
            rms_of[tid] = sqrtf(__fadd_rn(__fdiv_rn(ss, (float)D), a.eps));
        }
        __syncthreads();  // also: every lane has read the row before any lane writes it (out may be x)
        for (int pidx = tid; pidx < nrow * (int)half; pidx += 256) {
            const int lr = pidx / half;
            const uint32_t i = pidx % half;
            int64_t t = row0 + lr;
            const uint32_t r = (uint32_t)(t % a.shape[2]);
            t /= a.shape[2];
            const int64_t sb = (t / a.shape[1]) * a.ss[0] + (t % a.shape[1]) * a.ss[1] + r * a.ss[2];
            const int64_t db = (t / a.shape[1]) * a.ds[0] + (t % a.shape[1]) * a.ds[1] + r * a.ds[2];
            const float rms = rms_of[lr];
            const uint32_t d0 = a.mode == 0 ? i : 2 * i, d1 = a.mode == 0 ? i + half : 2 * i + 1;
            float x0 = __fmul_rn(__fdiv_rn(load_as_f32(a.src, sb + d0 * a.ss[3], a.src_dtype), rms),
                                 load_as_f32(a.norm_w, d0, a.norm_dtype));
            float x1 = __fmul_rn(__fdiv_rn(load_as_f32(a.src, sb + d1 * a.ss[3], a.src_dtype), rms),
                                 load_as_f32(a.norm_w, d1, a.norm_dtype));
            if (a.norm_b) {
                x0 = __fadd_rn(x0, load_as_f32(a.norm_b, d0, a.norm_dtype));
                x1 = __fadd_rn(x1, load_as_f32(a.norm_b, d1, a.norm_dtype));
            }
            x0 = round_through(x0, a.src_dtype);
            x1 = round_through(x1, a.src_dtype);
            float y0 = x0, y1 = x1;
            if (a.mode != 2) {
                const float c = a.cos[(a.pos0 + r) * half + i], s = a.sin[(a.pos0 + r) * half + i];
                y0 = __fsub_rn(__fmul_rn(x0, c), __fmul_rn(x1, s));
                y1 = a.mode == 0 ? __fadd_rn(__fmul_rn(x1, c), __fmul_rn(x0, s))
                                 : __fadd_rn(__fmul_rn(x0, s), __fmul_rn(x1, c));
            }
            store_from_f32(a.dst, db + d0 * a.ds[3], a.dst_dtype, y0);
            store_from_f32(a.dst, db + d1 * a.ds[3], a.dst_dtype, y1);
        }
        __syncthreads();  // rms_of is rewritten by the next group
    }
}

__global__ __launch_bounds__(256, 2) void norm_rope_rows_kernel(RopeRows a) {
    __shared__ NormWaveLds lds[4];
    __shared__ float rms_of[NORM_ROPE_MAX_ROWS];
    if (a.vec) norm_rope_rows_vec_any(a, &lds[threadIdx.x >> 6]);
    else norm_rope_rows_body(a, rms_of);
}

__device__ __forceinline__ void rope_rows_body(const RopeRows &a) {
    const uint32_t D = a.shape[3], half = D / 2;
    const int64_t per_row = a.mode == 2 ? D : half;
    const int64_t total = (int64_t)a.shape[0] * a.shape[1] * a.shape[2] * per_row;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const uint32_t i = (uint32_t)(idx % per_row);
        int64_t t = idx / per_row;
        const uint32_t r = (uint32_t)(t % a.shape[2]);
        t /= a.shape[2];
        const uint32_t h = (uint32_t)(t % a.shape[1]);
        const uint32_t b = (uint32_t)(t / a.shape[1]);
        const int64_t sb = b * a.ss[0] + h * a.ss[1] + r * a.ss[2];
        const int64_t db = b * a.ds[0] + h * a.ds[1] + r * a.ds[2];
        if (a.mode == 2) {
            store_from_f32(a.dst, db + i * a.ds[3], a.dst_dtype, load_as_f32(a.src, sb + i * a.ss[3], a.src_dtype));
            continue;
        }
        const float c = a.cos[(a.pos0 + r) * half + i], s = a.sin[(a.pos0 + r) * half + i];
        const uint32_t d0 = a.mode == 0 ? i : 2 * i, d1 = a.mode == 0 ? i + half : 2 * i + 1;
        const float x0 = load_as_f32(a.src, sb + d0 * a.ss[3], a.src_dtype);
        const float x1 = load_as_f32(a.src, sb + d1 * a.ss[3], a.src_dtype);
        // every product and sum is rounded on its own: this file is compiled with -ffp-contract=off
        const float y0 = __fsub_rn(__fmul_rn(x0, c), __fmul_rn(x1, s));
        const float y1 = a.mode == 0 ? __fadd_rn(__fmul_rn(x1, c), __fmul_rn(x0, s))
                                     : __fadd_rn(__fmul_rn(x0, s), __fmul_rn(x1, c));
        store_from_f32(a.dst, db + d0 * a.ds[3], a.dst_dtype, y0);
        store_from_f32(a.dst, db + d1 * a.ds[3], a.dst_dtype, y1);
    }
}

__global__ __launch_bounds__(256) void rope_rows_kernel(RopeRows a) {
    if (a.vec) rope_rows_vec_body(a);
    else rope_rows_body(a);
}

// Several row jobs in one launch (blockIdx.y picks the job): the rotation of q, the rotated keys and the values of
// one decode step are three tiny jobs whose launch cost exceeds their run time.
__global__ __launch_bounds__(256, 2) void row_jobs_kernel(RowJobs js) {
    __shared__ NormWaveLds lds[4];
    __shared__ float rms_of[NORM_ROPE_MAX_ROWS];
    const RopeRows &a = js.job[blockIdx.y];
    if (a.norm_w) {
        if (a.vec) norm_rope_rows_vec_any(a, &lds[threadIdx.x >> 6]);
        else norm_rope_rows_body(a, rms_of);
    } else {
        if (a.vec) rope_rows_vec_body(a);
        else rope_rows_body(a);
    }
}

void fill_row_job(RopeRows *out, const void *src, const int64_t ss[4], fhip_dtype src_dtype, void *dst, const int64_t ds[4],
                  fhip_dtype dst_dtype, const uint32_t shape[4], const float *cos, const float *sin, int64_t pos0, int mode,
                  const RowNorm *norm) {
    RopeRows &a = *out;
    a.src = src;
    a.dst = dst;
    for (int i = 0; i < 4; i++) {
        a.ss[i] = ss[i];
        a.ds[i] = ds[i];
        a.shape[i] = shape[i];
    }
    a.src_dtype = src_dtype;
    a.dst_dtype = dst_dtype;
    a.cos = cos;
    a.sin = sin;
    a.pos0 = pos0;
    a.mode = mode;
    a.norm_w = norm ? norm->weight : nullptr;
    a.norm_b = norm ? norm->bias : nullptr;
    a.norm_dtype = norm ? norm->dtype : FHIP_F32;
    a.eps = norm ? norm->eps : 0.0f;
    // the wide forms: consecutive elements, every row start a multiple of four elements from an address aligned to
    // four elements, on both sides; the tables (if used) 16-byte aligned
    const uint32_t D = shape[3];
    auto wide = [&](const void *p, const int64_t st[4], fhip_dtype t) {
        const uintptr_t step = (t == FHIP_F32 ? 4 : 2) * 4;
        if (D > 1 && st[3] != 1) return false;
        if (((uintptr_t)p % step) != 0) return false;
        for (int i = 0; i < 3; i++)
            if (shape[i] > 1 && st[i] % 4 != 0) return false;
        return true;
    };
    a.vec = D % 8 == 0 && D >= 8 && wide(src, ss, src_dtype) && wide(dst, ds, dst_dtype) &&
            (mode == 2 || (((uintptr_t)cos % 16) == 0 && ((uintptr_t)sin % 16) == 0));
    if (a.norm_w && !(D == 64 || D == 128 || D == 256)) a.vec = 0;  // the head dims the wide normalised form is built for
    // fewer than two full-size blocks per SIMD of a 256-CU chip: a quarter of the rows per block, four times the blocks
    const int64_t rows = (int64_t)shape[0] * shape[1] * shape[2];
    const int64_t full = D == 64 ? 32 : D == 128 ? 16 : 8;
    // a quarter of the rows per block below 2048 full blocks (an eighth measured slower: 33.8 against 31.9 us on a
    // 512-token prompt step whose full blocks took 35.9 us)
    a.few = a.norm_w && a.vec && rows < 2048 * full ? 4 : 1;
}

// rows per wavefront block of the wide normalised form (RPW in norm_rope_rows_vec_body)
static int norm_rows_per_wave(const RopeRows &a) {
    const int D = (int)a.shape[3];
    return (D == 64 ? 32 : D == 128 ? 16 : 8) / (a.few > 1 ? a.few : 1);
}

static int64_t job_blocks(const RopeRows &a) {
    const int64_t rows = (int64_t)a.shape[0] * a.shape[1] * a.shape[2];
    if (rows == 0 || a.shape[3] == 0) return 0;
    if (a.norm_w) {
        const int rpb = a.vec ? 4 * norm_rows_per_wave(a) : (a.shape[3] / 2 >= 256 ? 1 : 256 / (a.shape[3] / 2));
        return (rows + rpb - 1) / rpb;
    }
    const int64_t total = a.vec ? rows * (a.mode == 2 ? a.shape[3] / 4 : a.shape[3] / 8)
                                : rows * (a.mode == 2 ? a.shape[3] : a.shape[3] / 2);
    return (total + 255) / 256;
}

int launch_row_jobs(const RowJobs &js, hipStream_t stream) {
    if (js.n <= 0) return FHIP_OK;
    int64_t blocks = 0;
    for (int i = 0; i < js.n; i++) blocks = blocks > job_blocks(js.job[i]) ? blocks : job_blocks(js.job[i]);
    if (blocks == 0) return FHIP_OK;  // the bodies stride over their own work, so an over-sized grid.x is harmless
    hipLaunchKernelGGL(row_jobs_kernel, dim3((unsigned)(blocks < 65536 ? blocks : 65536), (unsigned)js.n), dim3(256), 0, stream, js);
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

int launch_rope_rows(const void *src, const int64_t ss[4], fhip_dtype src_dtype, void *dst, const int64_t ds[4],
                     fhip_dtype dst_dtype, const uint32_t shape[4], const float *cos, const float *sin, int64_t pos0,
                     int mode, const RowNorm *norm, hipStream_t stream) {
    RopeRows a;
    fill_row_job(&a, src, ss, src_dtype, dst, ds, dst_dtype, shape, cos, sin, pos0, mode, norm);
    const int64_t blocks = job_blocks(a);
    if (blocks == 0) return FHIP_OK;
    const dim3 grid((unsigned)(blocks < 65536 ? blocks : 65536));
    if (a.norm_w) hipLaunchKernelGGL(norm_rope_rows_kernel, grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(rope_rows_kernel, grid, dim3(256), 0, stream, a);
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

}  // namespace fhip
