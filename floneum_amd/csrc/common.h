// Internal declarations shared by the C-ABI layer and the kernel launchers.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include "../../include/fusor_hip.h"

namespace fhip {

// What every attention kernel receives: base pointers with the view offset already applied,
// element strides, and the mask description reduced to what the device needs.
struct AttnParams {
    const void *q, *k, *v;
    void *out;
    const void *mask;       // nullptr when there is no additive mask tensor
    const int32_t *kv_lens; // nullptr or [B]
    int64_t qs[4], ks[4], vs[4], os[4];
    int64_t ms0, ms1;       // mask strides: row (query for QK, batch for BATCH_KEY), key
    int32_t B, H, Hkv, G, Sq, Skv, D;
    int32_t mask_kind;      // fhip_mask_kind of `mask`
    int32_t analytic, causal;
    int64_t q_pos_offset, window;
    float scale;
    int32_t out_f32;        // 1: out is f32 although the inputs are 16-bit
    int32_t cus;            // compute units of the device the call runs on (launch planning)
    // split-KV decode only
    float *partials;        // [B, H, nsplit, D + 2] per-split (acc, m, l)
    int32_t chunk;          // keys per split
    int32_t nsplit;         // splits per (batch, kv head) over Skv
    int32_t dec_waves;      // wavefronts per workgroup of the 16-bit matrix-core decode variant (4 or 8)
    // Fused merge of the 16-bit matrix-core decode variant (no second kernel): the workgroups of a (batch, kv head)
    // unit run on one XCD, park their partials in that XCD's L2 and the last one to arrive merges them.
    int32_t dec_fused;        // 0: two kernels
    int32_t dec_unit_stride;  // floats between the partials of consecutive units (a multiple of 32: 128-byte lines)
    uint32_t dec_tag;         // unique to the call (20 bits are used): arrival counters need no clearing
    uint32_t *dec_counters;   // [units] arrival counters: tag | XCC id of the first arrival | arrivals
    size_t dec_counters_offset;  // host side: bytes from the workspace's start to the counters
    int32_t *dec_trip;        // host-visible word set when the workgroups of a unit turn out to run on different XCDs
    // host-side only (profiling hook).  Both set: the dispatch of the main kernel carries the two events, which then
    // hold its own begin and end timestamps.  Only main_done: recorded on the stream after the main kernel.
    hipEvent_t main_start, main_done;
    // Dense additive mask reduced to intervals (see mask_intervals.hip).  iv[r] = {lo, hi}: row r of the
    // mask is 0 on keys [lo, hi) and -inf elsewhere; r is the query row (FHIP_MASK_QK) or the batch
    // (FHIP_MASK_BATCH_KEY).  *iv_bad holds bad_tag when some row is NOT of that form.  A tiled kernel given
    // `iv` does nothing when *iv_bad == bad_tag; the kernel given `only_if_bad` does nothing when
    // *only_if_bad != bad_tag: exactly one of the two computes the result.
    const int2 *iv;
    // With iv_either set the f32-arithmetic tiled kernel (head_dim <= 64) serves the call whatever the scan found: it
    // masks by interval when *iv_bad != bad_tag and adds the mask values otherwise, and no second kernel is queued.
    int32_t iv_either;
    const int32_t *iv_bad;
    const int32_t *only_if_bad;
    // What the scan writes to *iv_bad when a row is not of that form: a value unique to the call, so that the word
    // needs no clearing beforehand (whatever the workspace held, it is not this call's tag, short of a 2^-32
    // coincidence that only costs the fast path).
    int32_t bad_tag;
    // Tiled f32 prefill only.  Workgroups are numbered longest first.  When the whole grid is resident at once
    // (two workgroups per CU) nothing is rebalanced at run time, so the second half of the numbers is walked
    // backwards: a CU's two workgroups are then a long and a short one.  0: off; else the number of CUs.
    int32_t snake_cus;
    // Tiled prefill kernels: keys split over pf_nsplit workgroups per query block (few query rows on a long
    // cache would otherwise occupy a fraction of the chip).  Split s takes keys [s * pf_chunk, (s + 1) * pf_chunk)
    // and parks (O unnormalised, m, l) per row in `partials` [B, H, Sq, pf_nsplit, pf_pitch]; a merge kernel follows.
    int32_t pf_nsplit, pf_chunk;
    int32_t pf_pitch;  // floats per (row, share) in `partials`: D + 2, or D + 4 where rows are written in 16-byte pieces
    int32_t pf_pack;   // tiled kernels, set by their launchers: query heads per workgroup of the packed form, or 0
    int32_t pf_rows64; // 16-bit tiled prefill at head_dim 128: the caller forced the 64-rows-per-wavefront form
};

// the key split of a tiled f32 prefill call (1 = none) and the scratch it needs
void prefill_f32_plan(int B, int H, int G, int Sq, int Skv, int D, bool causal_square, int compute_units, int *nsplit, int *chunk);
size_t prefill_f32_workspace_bytes(int B, int H, int Sq, int D, int nsplit);
// the same for the 16-bit matrix-core prefill kernel (256-row query blocks, one workgroup per CU)
void prefill_mfma_plan(int B, int H, int G, int Sq, int Skv, bool causal_square, int compute_units, int *nsplit, int *chunk);
// query heads that share one workgroup's K/V tiles (0: one head per workgroup)
int prefill_mfma_pack(int B, int H, int G, int Sq, int Skv, int compute_units);
size_t prefill_mfma_workspace_bytes(int B, int H, int Sq, int D, int nsplit);
// merges the key shares parked in p.partials (p.pf_nsplit, p.pf_pitch) into p.out
int launch_prefill_merge(const AttnParams &p, fhip_dtype dtype, hipStream_t stream);

// bytes of device scratch the interval form of a dense mask needs
size_t mask_intervals_bytes(int rows);
// fills iv[rows] from the mask described by p.mask / p.ms0 / p.ms1 / p.mask_kind and stores p.bad_tag in *bad if some
// row is not an interval (*bad is left alone otherwise: whatever it held is not this call's mark)
int launch_mask_intervals(const AttnParams &p, fhip_dtype dtype, int2 *iv, int32_t *bad, hipStream_t stream);

// writes get_mask's [rows, cols] tensor (0 / -inf bit patterns of `dtype`) into device memory; off = cols - rows
int launch_mask_build(void *out, fhip_dtype dtype, uint32_t rows, uint64_t cols, uint64_t off, int has_window,
                      uint64_t window, hipStream_t stream);

// layout of the fused split-KV merge in the workspace (false: the call takes the two-kernel form)
bool decode_fused_layout(const AttnParams &p, bool f32, int *unit_stride, size_t *counters_offset);
// writes the XCC id each of `workgroups` workgroups of a one-dimensional launch runs on
int launch_xcd_probe(uint8_t *out, int workgroups, hipStream_t stream);

// thread-local error text
void set_error(const char *fmt, ...);
int hip_fail(hipError_t e, const char *what);

#define FHIP_HIP_CHECK(expr)                                  \
    do {                                                      \
        hipError_t e__ = (expr);                              \
        if (e__ != hipSuccess) return fhip::hip_fail(e__, #expr); \
    } while (0)

// Launch of a call's main kernel: with both profiling events the dispatch itself is timestamped into them (what a
// profiler's kernel trace reports), otherwise a plain launch.
#define FHIP_LAUNCH_MAIN(kernel, grid, block, stream, p, ...)                                                    \
    do {                                                                                                         \
        if ((p).main_start && (p).main_done)                                                                     \
            hipExtLaunchKernelGGL(kernel, grid, block, 0, stream, (p).main_start, (p).main_done, 0, __VA_ARGS__); \
        else                                                                                                     \
            hipLaunchKernelGGL(kernel, grid, block, 0, stream, __VA_ARGS__);                                      \
    } while (0)
// after the main kernel: the stream marker of the older form of the hook (main_done alone)
#define FHIP_MARK_MAIN_DONE(p, stream)                                                                           \
    do {                                                                                                         \
        if ((p).main_done && !(p).main_start) FHIP_HIP_CHECK(hipEventRecord((p).main_done, stream));              \
    } while (0)

// launchers (each returns a status code, all asynchronous on `stream`)
int launch_generic(const AttnParams &p, fhip_dtype dtype, hipStream_t stream);
int launch_decode(const AttnParams &p, fhip_dtype dtype, hipStream_t stream);
int launch_prefill_mfma(const AttnParams &p, fhip_dtype dtype, hipStream_t stream);
// the same for head dims 160 / 192 / 224 / 256 (four wavefronts per workgroup, 128 query rows, 32-key tiles)
int launch_prefill_mfma_wide(const AttnParams &p, fhip_dtype dtype, hipStream_t stream);
void prefill_mfma_wide_plan(int B, int H, int G, int Sq, int Skv, bool causal_square, int compute_units, int *nsplit, int *chunk);
// head dims above 192 on 128-row workgroups of four wavefronts with 32 rows each (one per SIMD, software-pipelined)
bool prefill_mfma_rows32_takes(const AttnParams &p);
int launch_prefill_mfma_rows32(const AttnParams &p, fhip_dtype dtype, hipStream_t stream);
// head_dim 128 on 256-row workgroups of four wavefronts with 64 rows each (FHIP_KERNEL_PREFILL_MFMA_ROWS64: forced only)
bool prefill_mfma_rows64_takes(int D, float scale);
int launch_prefill_mfma_rows64(const AttnParams &p, fhip_dtype dtype, hipStream_t stream);
// f32 arithmetic on the f32 matrix cores; `dtype` is the tensors' storage type (16-bit rows are widened on load)
int launch_prefill_f32(const AttnParams &p, fhip_dtype dtype, hipStream_t stream);

// decode planning (host): keys per split and number of splits; `ragged`: per-batch key counts are given;
// `f32`: the tensors are f32 (vector variant) rather than 16-bit
void decode_plan(int B, int Hkv, int G, int Skv, int D, int compute_units, bool ragged, bool f32, int *chunk,
                 int *nsplit, int *waves);
size_t decode_workspace_bytes(int B, int H, int Hkv, int D, int nsplit);

// calibration (calibration.hip): the register-only matrix-core loop and the scratch it reports into
size_t calibration_mfma_bytes(int compute_units);
int launch_calibration_mfma(fhip_dtype dtype, int compute_units, int duty_percent, int rounds, int random_operands, void *scratch,
                            hipStream_t stream);
// steps of one matrix instruction and the companions `mix` names, one wavefront per SIMD; scratch as for the loop above
int launch_calibration_issue(int mix, int compute_units, int rounds, void *scratch, hipStream_t stream);

int launch_calibration_read(const void *src, size_t bytes, int compute_units, void *sink, hipStream_t stream);

// KV cache copies
int launch_copy_rows(const void *src, const int64_t sstride[4], void *dst, const int64_t dstride[4],
                     const uint32_t shape[4], int elem_bytes, hipStream_t stream);
int launch_fill_zero_bytes(void *dst, size_t bytes, hipStream_t stream);
int launch_fill_bytes(void *dst, int value, size_t bytes, hipStream_t stream);
int launch_fill_zero_rows(void *dst, const int64_t dstride[4], const uint32_t shape[4], int elem_bytes,
                          hipStream_t stream);

// Rotary embedding / type conversion of rows [B, heads, rows, D] from a strided source into a strided
// destination.  mode 0: pairs (i, i + D/2), 1: pairs (2i, 2i+1), 2: conversion only.  pos0 is the row
// of the cos/sin tables ([positions, D/2] f32) that row 0 uses.
// norm (nullable): RMS-normalise each row first with weight / bias [D] of norm->dtype, result rounded to
// src_dtype before the rotation.  Needs an even D.
struct RowNorm {
    const void *weight, *bias;
    fhip_dtype dtype;
    float eps;
};
// one row-wise job: rows of `src` rotated / normalised / converted into `dst` (what launch_rope_rows does)
struct RopeRows {
    const void *src;
    void *dst;
    int64_t ss[4], ds[4];
    uint32_t shape[4];  // [B, heads, rows, D]
    int32_t src_dtype, dst_dtype;
    const float *cos, *sin;
    int64_t pos0;       // table row of row 0
    int32_t mode;       // 0 normal, 1 interleaved, 2 convert only
    const void *norm_w, *norm_b;  // [D] weight (nullptr: no norm) and optional bias, of norm_dtype
    int32_t norm_dtype;
    float eps;
    int32_t vec;  // rows and pointers allow the 16-byte forms (set by fill_row_job)
    int32_t few;  // the wide normalised form with its rows per wavefront block divided by 1 or 4 (set by fill_row_job)
};
struct RowJobs {
    RopeRows job[3];
    int32_t n;
};
void fill_row_job(RopeRows *out, const void *src, const int64_t sstride[4], fhip_dtype src_dtype, void *dst,
                  const int64_t dstride[4], fhip_dtype dst_dtype, const uint32_t shape[4], const float *cos, const float *sin,
                  int64_t pos0, int mode, const RowNorm *norm);
// all jobs in ONE launch
int launch_row_jobs(const RowJobs &jobs, hipStream_t stream);
int launch_rope_rows(const void *src, const int64_t sstride[4], fhip_dtype src_dtype, void *dst,
                     const int64_t dstride[4], fhip_dtype dst_dtype, const uint32_t shape[4], const float *cos,
                     const float *sin, int64_t pos0, int mode, const RowNorm *norm, hipStream_t stream);

}  // namespace fhip
