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

// The normalised variant: a workgroup takes groups of rows; one lane per row folds the squares in the
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

__global__ __launch_bounds__(256) void norm_rope_rows_kernel(RopeRows a) {
    __shared__ float rms_of[NORM_ROPE_MAX_ROWS];
    norm_rope_rows_body(a, rms_of);
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

__global__ __launch_bounds__(256) void rope_rows_kernel(RopeRows a) { rope_rows_body(a); }

// Several row jobs in one launch (blockIdx.y picks the job): the rotation of q, the rotated keys and the values of
// one decode step are three tiny jobs whose launch cost exceeds their run time.
__global__ __launch_bounds__(256) void row_jobs_kernel(RowJobs js) {
    __shared__ float rms_of[NORM_ROPE_MAX_ROWS];
    const RopeRows &a = js.job[blockIdx.y];
    if (a.norm_w) norm_rope_rows_body(a, rms_of);
    else rope_rows_body(a);
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
}

static int64_t job_blocks(const RopeRows &a) {
    const int64_t rows = (int64_t)a.shape[0] * a.shape[1] * a.shape[2];
    if (rows == 0 || a.shape[3] == 0) return 0;
    if (a.norm_w) {
        const int rpb = a.shape[3] / 2 >= 256 ? 1 : 256 / (a.shape[3] / 2);
        return (rows + rpb - 1) / rpb;
    }
    const int64_t total = rows * (a.mode == 2 ? a.shape[3] : a.shape[3] / 2);
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
    if (a.norm_w) {
        const int64_t rows = (int64_t)shape[0] * shape[1] * shape[2];
        if (rows == 0 || shape[3] == 0) return FHIP_OK;
        const int rpb = shape[3] / 2 >= 256 ? 1 : 256 / (shape[3] / 2);
        const int64_t blocks = (rows + rpb - 1) / rpb;
        hipLaunchKernelGGL(norm_rope_rows_kernel, dim3((unsigned)(blocks < 65536 ? blocks : 65536)), dim3(256), 0, stream, a);
        FHIP_HIP_CHECK(hipGetLastError());
        return FHIP_OK;
    }
    const int64_t total = (int64_t)shape[0] * shape[1] * shape[2] * (mode == 2 ? shape[3] : shape[3] / 2);
    if (total == 0) return FHIP_OK;
    const int64_t blocks = (total + 255) / 256;
    hipLaunchKernelGGL(rope_rows_kernel, dim3((unsigned)(blocks < 65536 ? blocks : 65536)), dim3(256), 0, stream, a);
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

}  // namespace fhip
