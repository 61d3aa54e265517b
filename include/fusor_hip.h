/*
 * fusor_hip.h -- C ABI of the MI355X (gfx950) attention backend for fusor-ml.
 *
 * This is the boundary a fusor HIP backend crate binds with `unsafe extern "C"`; it replaces the
 * GPU arm of `fusor::Tensor<4,D>::flash_attention` (reference:
 * fusor-ml/fusor/src/composite/flash_attention.rs:52-73), i.e. the WGSL custom op
 * `fusor_core::Tensor::flash_attention` / `FlashAttentionOperation`
 * (fusor-ml/core/src/composite/flash_attention.rs:28-99, 442-557).
 *
 * Conventions
 *   - Plain pointers and sizes only.  Every function returns an `int` status (0 = FHIP_OK); the
 *     text of the last failure on the calling thread is available from fhip_last_error().
 *     Nothing throws or aborts across this boundary: the reference's `assert!` panics on shape
 *     errors (flash_attention.rs:94-99,153-172) become FHIP_ERR_INVALID_ARG with the same message.
 *   - Tensors are described the way fusor's kernels receive them: a device buffer plus
 *     {offset, shape, strides} in ELEMENT units (fusor-ml/types/src/layout.rs:88-129,
 *     fusor-ml/core/src/mir/inputs/tensor.rs:33-119).  Arbitrary strided views are accepted
 *     (narrowed KV-cache views, transposed Q/V, broadcast strides of 0 on inputs).
 *   - The library never allocates or frees caller tensors.  The output buffer and the workspace
 *     are supplied by the caller.  Launches are asynchronous on the given stream.
 *   - Re-entrant: the only mutable state lives in the handles (a device handle holds an atomic counter that
 *     numbers masked prefill calls, a KV cache its buffers) and in the thread-local error string.  The one
 *     file-scope object is the fixed device array behind fhip_flash_attention_noalloc (one copy per GPU, shared
 *     by that GPU's calls of that function only).  Calls on different streams may run concurrently from different
 *     threads, also on one device handle; one stream, one KV cache and one workspace are used by one thread at a
 *     time.
 */
#ifndef FUSOR_HIP_H
#define FUSOR_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status ---------------------------------------------------------------------------------- */
enum {
    FHIP_OK = 0,
    FHIP_ERR_INVALID_ARG = 1, /* what the reference panics on: shapes, divisibility, null pointers  */
    FHIP_ERR_UNSUPPORTED = 2, /* valid request with no kernel (e.g. head_dim > 512)                */
    FHIP_ERR_HIP = 3,         /* a HIP runtime call failed (reference: fusor::Error::Gpu,
                                 fusor-ml/fusor/src/lib.rs:391-403)                                */
    FHIP_ERR_WORKSPACE = 4    /* workspace missing or smaller than *_workspace_bytes reports       */
};

/* Message of the last non-zero status returned on this thread ("" if none).  Never NULL. */
const char *fhip_last_error(void);

typedef struct fhip_device fhip_device;
typedef struct fhip_stream fhip_stream;
typedef struct fhip_event fhip_event;

/* ---- element types (reference: DataTypeEnum, fusor-ml/core/src/tensor.rs:110-134) ------------ */
typedef enum { FHIP_F32 = 0, FHIP_F16 = 1, FHIP_BF16 = 2 } fhip_dtype;

/* ---- mask layout (reference: enum MaskKind, fusor flash_attention.rs:11-19) ------------------ */
typedef enum {
    FHIP_MASK_NONE = 0,
    FHIP_MASK_QK = 1,       /* [q_seq_len, kv_seq_len], shared by every (batch, head)            */
    FHIP_MASK_BATCH_KEY = 2 /* [batch, kv_seq_len], broadcast over heads and queries             */
} fhip_mask_kind;

/* Rank-4 strided view [batch, heads, seq, head_dim].  Element (b,h,s,d) lives at
 * ptr[offset + b*stride[0] + h*stride[1] + s*stride[2] + d*stride[3]]  (element units). */
typedef struct {
    void *ptr;
    uint64_t offset;
    uint32_t shape[4];
    int64_t stride[4];
} fhip_tensor4;

/* Rank-2 strided view (the mask). */
typedef struct {
    void *ptr;
    uint64_t offset;
    uint32_t shape[2];
    int64_t stride[2];
} fhip_tensor2;

/* Optional analytic description of the mask.  It NEVER replaces semantics: when `enabled`, the
 * caller promises that the additive mask it would otherwise pass is exactly
 *     mask[i][j] = -inf  if  j > i + q_pos_offset                      (causal part)
 *                  -inf  if  window > 0 and j + window <= i + q_pos_offset   (sliding part)
 *                  0     otherwise
 * which is what MaskCache::get_mask builds (fusor-ml/fusor/src/cache/mask_cache.rs:36-116) with
 * q_pos_offset = the left padding it computes.  The kernels then skip fully masked key tiles
 * and never read a mask tensor.  `mask.ptr` must be NULL when this is enabled. */
typedef struct {
    int32_t enabled;
    int32_t causal;       /* 0: no causal part (only the window, if any)                          */
    int64_t q_pos_offset; /* key index the first query row may still see: kv_seq_len - q_seq_len
                             for a chunk appended to a cache                                      */
    int64_t window;       /* 0 = none                                                             */
} fhip_analytic_mask;

/* Arguments of one attention call.  Zero-initialise, then fill. */
typedef struct {
    fhip_tensor4 q;   /* [B, H,   Sq,  D] */
    fhip_tensor4 k;   /* [B, Hkv, Skv, D] */
    fhip_tensor4 v;   /* [B, Hkv, Skv, D] */
    fhip_tensor4 out; /* [B, H,   Sq,  D]  fresh buffer of Q's shape (reference: core :505-507)  */
    fhip_dtype dtype;     /* element type of q, k, v and the mask                                  */
    fhip_dtype out_dtype; /* the reference returns Q's dtype; FHIP_F32 is also accepted for f16/bf16
                             inputs (accumulators are f32 either way, core :186-203,323-327)       */
    float scale;
    fhip_mask_kind mask_kind;
    fhip_tensor2 mask;
    fhip_analytic_mask analytic;
    /* Optional device array of B int32: keys j >= kv_lens[b] are masked for batch b.  Equivalent
     * to a 0 / -inf BatchKeyMask; it exists so a ragged batch needs no [B,Skv] mask tensor. */
    const int32_t *kv_lens;
    void *workspace; /* device scratch, >= fhip_flash_attention_workspace_bytes(), 16-byte aligned,
                        contents irrelevant; may be NULL when the size query reports 0.  Calls that
                        share a workspace must not overlap.  Split-KV decode needs it for its partial
                        results.  A prefill call with a mask TENSOR uses it to reduce the mask to one
                        visible interval per row on the device (every mask fusor builds, and every
                        padding mask, has that form) and then runs the tiled kernel; a mask that is
                        not of that form, or a call that brings no workspace, is served by a kernel
                        that adds the mask values like the reference.  A prefill call of few query rows
                        on a long cache uses it to split the keys over workgroups (the largest split
                        whose partial results fit); without it the call runs unsplit.                                       */
    size_t workspace_bytes;
    int32_t force_kernel; /* 0 = choose; otherwise a fhip_kernel_id (testing / benchmarking)       */
    /* Optional profiling hook: when non-NULL the event is recorded on the stream right after the
     * main kernel of the call (before the split-KV combine pass, if there is one), so a benchmark
     * can time that kernel alone with HIP events. */
    fhip_event *main_kernel_done;
    /* With main_kernel_done: when non-NULL too, the main kernel's dispatch itself carries the two events
     * and they hold its begin and end as the command processor stamps them; fhip_event_elapsed_ms(start,
     * done) is then the kernel's own duration, the figure a profiler's kernel trace gives.  A call that runs
     * no attention kernel (no output element, or no key) records start and then done on the stream.  Such a
     * dispatch cannot be recorded into a graph: with main_kernel_start set, a call on a stream that is being
     * captured fails with FHIP_ERR_UNSUPPORTED (main_kernel_done alone may be captured). */
    fhip_event *main_kernel_start;
    /* Optional, with a mask tensor: the table fhip_mask_intervals computed for exactly this mask view.  The tiled
     * prefill kernels then skip the scan of the mask (one launch and one pass over the tensor per call) and need no
     * workspace for it.  For masks that do not change between calls: one mask tensor serves every layer of a forward
     * pass, and MaskCache keeps its tensors for its lifetime.  The caller vouches that the mask's contents are what
     * they were when the table was computed; decode calls ignore it. */
    const void *mask_intervals;
} fhip_attn_args;

typedef enum {
    FHIP_KERNEL_AUTO = 0,
    FHIP_KERNEL_GENERIC = 1,     /* any dtype, any strides, any mask; one wavefront per query row   */
    FHIP_KERNEL_PREFILL_MFMA = 2,/* f16/bf16, head_dim a multiple of 8 up to 256, LDS-tiled MFMA (64 / 96 / 128 on
                                    256-row workgroups, the others on the wide-head form); masks by interval
                                    (analytic, kv_lens, or a mask tensor reduced on the device) */
    FHIP_KERNEL_PREFILL_F32 = 3, /* f32 arithmetic on the f32 MFMA, LDS-tiled: f32 tensors, and 16-bit tensors
                                    (widened on load) the kernel above does not take; head_dim multiple of
                                    4 up to 256; masks by interval or, up to head_dim 128, added as they are */
    FHIP_KERNEL_DECODE_SPLITKV = 4,/* 1..4 query rows per sequence, head_dim multiple of 8 up to 256: split-KV
                                      streaming + LSE combine.  Matrix cores at every head_dim that is a multiple
                                      of 32 up to 256 (the 16-bit or the f32 instruction, by the tensors' type;
                                      f32 at 224 / 256 from five columns per KV head on), vector units otherwise.  At the matrix-core head dims
                                      more rows ride along while rows x GQA group <= 32 (16 above head_dim 128;
                                      f32 tensors: 64 up to head_dim 192, 32 above): an 8-token draft on a 4-way
                                      GQA model                                                               */
    FHIP_KERNEL_PREFILL_MFMA_ROWS64 = 5 /* only as force_kernel, never chosen: FHIP_KERNEL_PREFILL_MFMA's calls at
                                      head_dim 128 on its other form, four wavefronts of 64 query rows per workgroup
                                      (one per SIMD, half the LDS operand reads per matrix instruction, keys never split
                                      over workgroups).  Same results; 1-3 % slower than the 256-row form of eight
                                      wavefronts on this chip, whose matrix kernels are bound by power.  Kept selectable
                                      for measurement (bench.py --config C3R)                                  */
} fhip_kernel_id;


typedef struct {
    char name[128];
    char arch[64];
    int32_t compute_units;
    int32_t wavefront_size;
    int32_t clock_khz;
    int32_t memory_clock_khz;
    int32_t memory_bus_bits;
    uint64_t total_memory;
    uint64_t lds_per_cu;
    uint64_t l2_bytes;
} fhip_device_info;

/* ---- device / stream / memory: the minimal backend a fusor HIP crate owns ---------------------
 * Replaces what fusor_core::Device does for WGPU (fusor-ml/core/src/device.rs:89-354): pick an
 * adapter, create buffers, upload (`Tensor::new`, core/src/tensor.rs) and read back
 * (`as_slice`, core/src/tensor.rs:797-896). */
int fhip_device_count(int32_t *count);
int fhip_device_create(int32_t ordinal, fhip_device **out);
int fhip_device_destroy(fhip_device *dev);
int fhip_device_get_info(fhip_device *dev, fhip_device_info *info);

int fhip_stream_create(fhip_device *dev, fhip_stream **out);
int fhip_stream_destroy(fhip_stream *s);
int fhip_stream_synchronize(fhip_stream *s);

int fhip_malloc(fhip_device *dev, size_t bytes, void **out);
int fhip_free(fhip_device *dev, void *ptr);
int fhip_memcpy_h2d(fhip_stream *s, void *dst, const void *src, size_t bytes);
int fhip_memcpy_d2h(fhip_stream *s, void *dst, const void *src, size_t bytes); /* synchronises */
int fhip_memcpy_d2d(fhip_stream *s, void *dst, const void *src, size_t bytes);
int fhip_memset(fhip_stream *s, void *dst, int value, size_t bytes); /* a fill kernel: may be recorded into a graph */

/* Stream capture.  A decode step is a handful of short launches (rope, cache write, attention, merge), so a
 * serving loop is bound by launch cost; everything this library queues between begin and end is recorded
 * into one graph instead of running, and fhip_graph_launch replays it with a single submission.  All entry
 * points that take a stream can be captured EXCEPT those that may allocate or synchronise: fhip_malloc /
 * fhip_free, fhip_memcpy_d2h, fhip_stream_synchronize, fhip_kv_cache_append* when the cache has to grow.
 * Pointers and shapes are frozen at capture time; what may change between replays is the CONTENT of device
 * memory, e.g. the int32 kv_lens a ragged decode call reads, the new rows, the cache itself.
 * (The reference has no counterpart: WGPU command buffers are rebuilt every step.) */
typedef struct fhip_graph fhip_graph;
int fhip_stream_begin_capture(fhip_stream *s);
int fhip_stream_end_capture(fhip_stream *s, fhip_graph **out);
int fhip_graph_launch(fhip_graph *g, fhip_stream *s);
int fhip_graph_destroy(fhip_graph *g);

/* HIP events on a library stream (timing in benchmarks; the reference has no GPU timers). */
int fhip_event_create(fhip_device *dev, fhip_event **out);
int fhip_event_destroy(fhip_event *e);
int fhip_event_record(fhip_event *e, fhip_stream *s);
int fhip_event_synchronize(fhip_event *e);
int fhip_event_elapsed_ms(fhip_event *start, fhip_event *stop, float *ms);

/* ---- attention ------------------------------------------------------------------------------ */

/* Host-only check of everything the reference asserts plus pointer/stride sanity.  Touches no
 * GPU.  Same status and message fhip_flash_attention would return. */
int fhip_flash_attention_validate(const fhip_attn_args *args);

/* Which kernel fhip_flash_attention will run for these arguments (host-only).  For a prefill call
 * with a mask tensor and a sufficient workspace in `args` this names the tiled kernel, which runs if
 * the mask turns out to be made of intervals (decided on the device) and otherwise hands over, inside
 * the same call, to the kernel that adds the mask values one by one (the mask-adding form of the
 * f32-arithmetic tiled kernel up to head_dim 128, the general kernel above; at head_dim <= 64 the
 * f32-arithmetic tiled kernel holds both forms and nothing is handed over); without the workspace it
 * names that kernel.  The answer does not depend on the device: how a kernel splits its work over the
 * compute units is planned inside the call, and fhip_flash_attention_workspace_bytes takes their number
 * because the scratch for those splits does. */
int fhip_flash_attention_select(const fhip_attn_args *args, int32_t *kernel_id);

/* Bytes of device workspace the call needs (0 for the single-pass kernels).  `compute_units`
 * is fhip_device_info.compute_units (split count depends on it). */
int fhip_flash_attention_workspace_bytes(const fhip_attn_args *args, int32_t compute_units, size_t *bytes);

/* out = softmax(q k^T * scale + mask) v with GQA head mapping kv_head = head / (H / Hkv).
 * Replaces fusor_core::Tensor::flash_attention (core/src/composite/flash_attention.rs:28-52) and,
 * for FHIP_MASK_BATCH_KEY, the composite fallback fusor takes on GPU (fusor
 * flash_attention.rs:61-72).  Asynchronous on `s`.
 * Rows whose keys are all masked come out NaN (0/0, as in the reference).  Tensors without elements
 * are valid: with no output element nothing runs; with no key (Skv == 0) the output is all zeros, which
 * is what the reference's [Sq, 0] x [0, D] product gives (fusor flash_attention.rs:141-199). */
int fhip_flash_attention(fhip_stream *s, const fhip_attn_args *args);

/* How a call would run on the split-KV decode kernels (for tests and benchmarks; no counterpart in the reference).
 * is_decode 0: another kernel takes the call and the other fields are 0.  Otherwise: the cache is streamed by
 * `nsplit` workgroups of `wavefronts` wavefronts per (batch, kv head, column block), `chunk` keys each, and the call
 * is `kernels` launches: 1 when nothing is split or the splits are merged inside the main kernel (equal-length
 * batches with 2 to 8 splits on the matrix-core variants, when the device deals the workgroups of a launch to its
 * XCDs round-robin so that the splits of a unit can share an XCD's L2), else 2 (a log-sum-exp merge kernel follows). */
typedef struct {
    int32_t is_decode;
    int32_t nsplit;
    int32_t chunk;
    int32_t wavefronts;
    int32_t kernels;
} fhip_decode_plan_info;
int fhip_flash_attention_decode_plan(fhip_stream *s, const fhip_attn_args *args, fhip_decode_plan_info *info);

/* fhip_flash_attention for callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments and same kernels,
 * but the workspace is a fixed array of FHIP_NOALLOC_WORKSPACE_BYTES of device
 * memory that the library holds on every GPU it is used on until the process ends; args->workspace and
 * args->workspace_bytes are ignored.  Neither this function nor anything it calls allocates or frees memory.
 * Only what a call cannot do without must fit the array: the split-KV partials of a decode call and the interval
 * table of a mask tensor (otherwise FHIP_ERR_WORKSPACE, and nothing runs).  The key split of a tiled prefill call
 * (few query rows on a long cache) is optional: it takes the largest split whose partial results fit, so such a call
 * may run with fewer shares than fhip_flash_attention_workspace_bytes plans, or unsplit (same results to the
 * stated tolerance).  Results are bit for bit those of fhip_flash_attention with a workspace of
 * FHIP_NOALLOC_WORKSPACE_BYTES.  All calls on one GPU share that GPU's array: two of them must not overlap in time
 * (one stream, or ordered by events); nothing in it has to be cleared between calls. */
#define FHIP_NOALLOC_WORKSPACE_BYTES (32u << 20)
int fhip_flash_attention_noalloc(fhip_stream *s, const fhip_attn_args *args);

/* Calibration for benchmarks (no counterpart in the reference): what the matrix cores deliver with nothing else
 * in the way.  One wavefront per SIMD of every compute unit runs `rounds` rounds of 32 v_mfma_f32_32x32x16
 * instructions (the instruction and per-tile count of the prefill kernel's matrix phase) on operands held in
 * registers: no LDS, no memory traffic, no vector work.  `random_operands` != 0: pseudo-random values in (-2, 2);
 * 0: all zero (no data toggling).  `duty_percent` (40..100): the share of the time the matrix pipe is kept busy
 * (the wavefront sleeps in between).  FLOPs per launch = 4 * compute_units * rounds * 32 * 32768.  `scratch`
 * (device, 16-byte aligned, compute_units * 1040 bytes) receives compute_units * 256 floats nobody needs and then,
 * per compute unit, two uint64: the shader-clock cycles and the 100 MHz wall-clock ticks its workgroup ran (their
 * ratio * 0.1 = the clock in GHz the chip held under this load).  `rounds` is at most
 * FHIP_CALIBRATION_MFMA_MAX_ROUNDS (about a second of matrix work).  Asynchronous on `s`. */
#define FHIP_CALIBRATION_MFMA_MAX_ROUNDS 2000000
int fhip_calibration_mfma(fhip_stream *s, fhip_dtype dtype, int32_t random_operands, int32_t duty_percent, int32_t rounds,
                          void *scratch, size_t scratch_bytes);

/* Calibration for benchmarks (no counterpart in the reference): what ONE wavefront per SIMD can issue beside its
 * matrix instructions.  A wavefront issues in order; a kernel that runs a single wavefront per SIMD (the prefill
 * kernel of head dims above 192, whose Q and O^T of 32 rows leave no registers for a second one) pays in full for
 * whatever does not fit into the 32 cycles the matrix pipe is busy with one v_mfma_f32_32x32x16.  One workgroup of
 * four wavefronts per compute unit runs `rounds` rounds of 16 steps, a step being one such instruction (f16,
 * independent accumulators) and the companions `mix` names:
 *   0 nothing; 1 nothing, and every matrix instruction depends on the one before; 2 four v_fma; 3 eight v_fma;
 *   4 four v_exp; 5 four scalar adds; 6 one ds_read_b128 that is the matrix operand eight steps later;
 *   7 as 6 and two more ds_read_b128; 8 two ds_read_b64_tr_b16 whose values a vector instruction takes eight steps
 *   later; 9 as 6 and 8 together; 10 as 9 and fma, exp2, add (the mix of the prefill kernel's softmax steps);
 *   11 two ds_read_b128 and fma, exp2, add; 12 two ds_read_b128, every other step a transposing read and every fourth
 *   a 16-byte LDS write (11 and 12: the steps of a kernel whose workgroup transposes a tile once for all its wavefronts).
 * `scratch` and what it receives are as for fhip_calibration_mfma: per compute unit the shader-clock cycles and the
 * 100 MHz wall-clock ticks of its workgroup; cycles / (16 * rounds) = cycles per step.  Asynchronous on `s`. */
#define FHIP_CALIBRATION_ISSUE_MIXES 13
int fhip_calibration_issue(fhip_stream *s, int32_t mix, int32_t rounds, void *scratch, size_t scratch_bytes);

/* Calibration for benchmarks (no counterpart in the reference): where the workgroups of a launch run.  A
 * one-dimensional launch of `workgroups` workgroups (64 lanes each) stores, per workgroup, the id of the XCD it ran
 * on (the XCC_ID hardware register) into the device bytes `out` (one per workgroup).  The split-KV decode kernels
 * that merge their splits inside the kernel rely on workgroups with the same number modulo 8 sharing an XCD; this
 * shows the dealing they rely on (the library checks it itself when a device handle is created).  Asynchronous on `s`. */
int fhip_calibration_xcd_map(fhip_stream *s, uint32_t workgroups, void *out, size_t out_bytes);

/* Calibration for benchmarks (no counterpart in the reference): a kernel that does nothing but read `bytes` of
 * device memory at `src` (16-byte aligned) once, with 16-byte non-temporal loads, eight in flight per lane: the
 * rate a streaming kernel of this shape can reach at most.  `scratch`: device memory of at least
 * compute_units * 32 bytes (nothing of interest is written there).  Asynchronous on `s`. */
int fhip_calibration_read(fhip_stream *s, const void *src, size_t bytes, void *scratch, size_t scratch_bytes);

/* ---- masks: host builders, bit-exact with the reference ---------------------------------------
 * `out` is host memory of the given dtype (f32: 0x00000000 / 0xFF800000; f16: 0x0000 / 0xFC00;
 * bf16: 0x0000 / 0xFF80), row-major contiguous. */

/* AttentionMask::causal (fusor-ml/fusor/src/cache/attention_mask.rs:26-46): [n, n]. */
int fhip_mask_causal(fhip_dtype dtype, uint32_t seq_len, void *out);
/* MaskCache::create_sliding_window_mask (fusor-ml/fusor/src/cache/mask_cache.rs:88-116): [n, n]. */
int fhip_mask_sliding_window(fhip_dtype dtype, uint32_t seq_len, uint64_t window, void *out);
/* MaskCache::get_mask (mask_cache.rs:36-86): shape [seq_len, offset' + seq_len] where
 * offset' = has_window ? min(seqlen_offset, window.saturating_sub(seq_len)) : seqlen_offset. */
int fhip_mask_get_mask_shape(uint32_t seq_len, uint64_t seqlen_offset, int32_t has_window,
                             uint64_t window, uint32_t *rows, uint64_t *cols);
int fhip_mask_get_mask(fhip_dtype dtype, uint32_t seq_len, uint64_t seqlen_offset,
                       int32_t has_window, uint64_t window, void *out);
/* The same tensor written by a kernel into device memory ([rows, cols] of fhip_mask_get_mask_shape, row-major):
 * no O(seq_len^2) host loop, no upload.  seqlen_offset = 0 without a window gives AttentionMask::causal,
 * with one MaskCache::create_sliding_window_mask.  Asynchronous on `s`. */
int fhip_mask_get_mask_device(fhip_stream *s, fhip_dtype dtype, uint32_t seq_len, uint64_t seqlen_offset,
                              int32_t has_window, uint64_t window, void *out_device);
/* The analytic descriptor equal to get_mask(seq_len, seqlen_offset, window) (no tensor built). */
/* The interval form of a mask tensor: for every row the run of keys where the mask is 0, if the row is zeros on one run
 * of keys and -inf elsewhere (every mask MaskCache::get_mask builds, padding masks, block-diagonal masks), and a mark
 * in the table's first word if some row is anything else (then calls that carry the table add the mask values like
 * the reference, as they would have without it).  What fhip_flash_attention computes per call from a mask tensor and
 * its workspace, computed once here: `table` is device memory of fhip_mask_intervals_bytes(mask->shape[0]) bytes,
 * 16-byte aligned, to be passed as fhip_attn_args.mask_intervals together with the same mask view.  No counterpart in
 * the reference.  Asynchronous on `s`. */
int fhip_mask_intervals_bytes(uint32_t rows, size_t *bytes);
int fhip_mask_intervals(fhip_stream *s, const fhip_tensor2 *mask, fhip_dtype dtype, void *table, size_t table_bytes);

int fhip_mask_get_analytic(uint32_t seq_len, uint64_t seqlen_offset, int32_t has_window,
                           uint64_t window, fhip_analytic_mask *out);

/* ---- growable KV cache on the device -----------------------------------------------------------
 * Replaces fusor::cache::KvCache / TensorCache for rank-4 [B, Hkv, seq, D] tensors concatenated
 * along dim 2 (fusor-ml/fusor/src/cache/kv_cache.rs:13-68, tensor_cache.rs:9-124; kalosm-llama
 * uses concat dim 2, models/kalosm-llama/src/raw/cache.rs:7).  Same observable behaviour:
 * first append stores the tensor, later appends grow the allocation to the next power of two and
 * write the new rows in place, the returned view is the valid prefix (stride[1] = allocated *
 * D), and once max_sequence_len would be exceeded only the last max_sequence_len positions are
 * kept.  Unlike the reference, growth copies once, in-place appends copy only the new rows, and a full
 * cache slides through a buffer of 2 * max_sequence_len rows (the returned view then has stride[1] =
 * 2 * max_sequence_len * D and a moving offset) instead of being re-concatenated on every append. */
typedef struct fhip_kv_cache fhip_kv_cache;
int fhip_kv_cache_create(fhip_device *dev, fhip_dtype dtype, uint64_t max_sequence_len, fhip_kv_cache **out);
int fhip_kv_cache_destroy(fhip_kv_cache *c);
/* TensorCache::reset (tensor_cache.rs:39-43): the cache is empty again.  Its buffers stay with it and serve the next
 * sequence's first buffers if they are large enough (no hipMalloc / hipFree per sequence); fhip_kv_cache_destroy frees
 * them.  Views returned before the reset are dead, and the next append must be ordered after the work that read them
 * (the same stream, or an event), as that work may still be running when reset returns. */
int fhip_kv_cache_reset(fhip_kv_cache *c);
int fhip_kv_cache_current_seq_len(const fhip_kv_cache *c, uint64_t *len);
int fhip_kv_cache_allocated_seq_len(const fhip_kv_cache *c, uint64_t *len);
/* k_new, v_new: [B, Hkv, n, D] strided device views of the cache dtype.  On return k_all/v_all
 * describe the cached keys/values including the new rows (views into cache-owned memory, valid
 * until the next append/reset/destroy: an append that grows the allocation, and the first one that
 * makes a full cache slide, move the rows to new buffers and free the old ones).  An append that
 * fails leaves the cache as it was. */
int fhip_kv_cache_append(fhip_kv_cache *c, fhip_stream *s, const fhip_tensor4 *k_new,
                         const fhip_tensor4 *v_new, fhip_tensor4 *k_all, fhip_tensor4 *v_all);

/* ---- rotary position embedding, fused with its destination --------------------------------------
 * The step right before attention in kalosm-llama (models/kalosm-llama/src/raw/attention_layer.rs:
 * 272-278, raw/rope.rs:86-111): q and k are cast to f32, rotated with the [positions, head_dim/2]
 * cos/sin tables of fusor::RopeCache (fusor-ml/fusor/src/composite/rope.rs:180-265), cast back, and k,
 * v are appended to the cache.  Here the rotation, the casts and the cache write are one pass:
 * arithmetic in f32 with one rounding per operation as on the reference's CPU path (rope.rs:46-137),
 * results rounded to nearest even into the destination type. */
typedef struct {
    const float *cos;    /* device, [table_rows, head_dim/2] f32 row-major (RopeCache::cos)           */
    const float *sin;    /* device, same shape (RopeCache::sin)                                        */
    uint64_t table_rows;
    uint64_t start_pos;  /* table row used by sequence position 0 of the tensor (RopeCache::forward)  */
    int32_t interleaved; /* 0: pairs (i, i + head_dim/2)  (rope, rope_normal_fused)
                            1: pairs (2i, 2i + 1)         (rope_interleaved, rope_fused)              */
} fhip_rope_tables;

/* out = rope(x): x, out [B, heads, seq, head_dim] strided device views of x_dtype / out_dtype; out may
 * be x itself.  Replaces Tensor::rope_normal_fused / rope_fused (rope.rs:139-175). */
int fhip_rope(fhip_stream *s, const fhip_rope_tables *rope, const fhip_tensor4 *x, fhip_dtype x_dtype,
              const fhip_tensor4 *out, fhip_dtype out_dtype);

/* fhip_kv_cache_append with the new keys rotated and both tensors converted from in_dtype to the
 * cache's type on the way in (no rotated copy of k, no separate cast pass). */
int fhip_kv_cache_rope_append(fhip_kv_cache *c, fhip_stream *s, const fhip_rope_tables *rope, const fhip_tensor4 *k_new,
                              const fhip_tensor4 *v_new, fhip_dtype in_dtype, fhip_tensor4 *k_all,
                              fhip_tensor4 *v_all);

/* ---- q / k RMS-norm fused into the rotation ------------------------------------------------------
 * Blocks with attention_q_norm / attention_k_norm (models/kalosm-llama/src/raw/attention_layer.rs:
 * 229-235,251-257) normalise every [head_dim] row of q and k before the rotation:
 * RmsNorm::forward_generic_4d (fusor-ml/fusor/src/layers/rms_norm.rs:122-133), i.e. in f32
 *   n = x / sqrt(mean(x * x) + eps) * weight (+ bias)
 * with the reference's operation order and its left-to-right sum (rms_norm_fused_cpu_impl,
 * fusor-ml/fusor/src/composite/normalization.rs:351-407), rounded to x's element type (the norm
 * returns a tensor of that type), then rotated as fhip_rope does. */
typedef struct {
    const void *weight; /* device, [head_dim] contiguous (RmsNorm::weight)                            */
    const void *bias;   /* device, [head_dim] contiguous, or NULL (RmsNorm::bias)                     */
    fhip_dtype dtype;   /* element type of weight and bias                                            */
    float eps;
} fhip_rms_norm;

/* out = rope(rms_norm(x)); arguments as fhip_rope.  rope == NULL: the norm alone. */
int fhip_norm_rope(fhip_stream *s, const fhip_rms_norm *norm, const fhip_rope_tables *rope, const fhip_tensor4 *x,
                   fhip_dtype x_dtype, const fhip_tensor4 *out, fhip_dtype out_dtype);

/* fhip_kv_cache_rope_append with the new keys normalised before they are rotated (the values are only
 * converted, as before). */
int fhip_kv_cache_norm_rope_append(fhip_kv_cache *c, fhip_stream *s, const fhip_rms_norm *k_norm,
                                   const fhip_rope_tables *rope, const fhip_tensor4 *k_new, const fhip_tensor4 *v_new,
                                   fhip_dtype in_dtype, fhip_tensor4 *k_all, fhip_tensor4 *v_all);

/* One decode (or prefill) step's preparation in ONE launch: q_out = rope(norm(q)), and the new keys / values
 * appended as fhip_kv_cache_norm_rope_append does (q_norm / k_norm may be NULL: no norm).  Three tiny row-wise
 * jobs whose launch cost exceeds their run time; bit-identical to the separate calls.  No counterpart in the
 * reference, which runs these as a dozen tensor ops (models/kalosm-llama/src/raw/attention_layer.rs:217-280,
 * 400-420). */
int fhip_kv_cache_qkv_rope_append(fhip_kv_cache *c, fhip_stream *s, const fhip_rms_norm *q_norm,
                                  const fhip_rms_norm *k_norm, const fhip_rope_tables *rope, const fhip_tensor4 *q,
                                  fhip_dtype q_dtype, const fhip_tensor4 *q_out, fhip_dtype q_out_dtype,
                                  const fhip_tensor4 *k_new, const fhip_tensor4 *v_new, fhip_dtype in_dtype,
                                  fhip_tensor4 *k_all, fhip_tensor4 *v_all);

/* Library version string, e.g. "fusor-hip 0.1 (gfx950)". */
const char *fhip_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FUSOR_HIP_H */
