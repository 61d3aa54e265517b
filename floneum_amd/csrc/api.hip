// C-ABI layer: handles, argument validation, kernel selection and dispatch, host mask builders,
// device KV cache.  Everything here is host code; kernels live in the attn_*.hip files.
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <new>

#include "common.h"

// Workspace of fhip_flash_attention_noalloc: device memory the library itself holds, so that the call needs no
// allocation by anyone.  Each GPU the library runs on has its own copy of the array at its own address, looked
// up once per device in fhip_device_create (the name below is only a host-side handle of the symbol, not a
// device address).  Its contents are whatever the last call left: every user of the workspace (split-KV
// partials, mask intervals and their per-call mark, prefill key shares) writes what it reads, so nothing has
// to start at zero.
constexpr size_t STATIC_WORKSPACE_BYTES = (size_t)FHIP_NOALLOC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_WORKSPACE_BYTES];

struct fhip_device {
    int ordinal;
    hipDeviceProp_t prop;
    void *scratch_ptr;  // this device's address of `scratch`
    // Source of the per-call marks of masked prefill calls (AttnParams::bad_tag): the one piece of state a device
    // handle changes after its creation.
    std::atomic<uint32_t> next_tag;
    // The fused split-KV merge needs workgroups L of a one-dimensional launch with the same L % 8 to share an XCD (and
    // with it an L2).  Probed once per handle.  `trip` is a word of pinned host memory the decode kernels set when the
    // workgroups of a unit find themselves on different XCDs all the same: the next decode call then fails once and the
    // form stays off for the handle.
    std::atomic<bool> xcd_grouped;
    int32_t *trip_host, *trip_dev;
};

// Do workgroups with the same number modulo 8 run on one XCD?  (The hardware deals the workgroups of a launch to its
// XCDs round-robin in launch order, starting wherever the previous launch of the queue left off: true for 8, 4, 2 or 1
// XCDs per device.)
static void probe_xcd_grouping(fhip_device *d) {
    d->xcd_grouped.store(false);
    d->trip_host = d->trip_dev = nullptr;
    constexpr int N = 4096;
    uint8_t *dev_ids = nullptr;
    uint8_t ids[N];
    if (hipMalloc((void **)&dev_ids, N) != hipSuccess) return;
    bool ok = fhip::launch_xcd_probe(dev_ids, N, nullptr) == FHIP_OK && hipMemcpy(ids, dev_ids, N, hipMemcpyDeviceToHost) == hipSuccess;
    (void)hipFree(dev_ids);
    for (int i = 0; ok && i < N; i++) ok = ids[i] < 16 && ids[i] == ids[i & 7];
    if (!ok) return;
    if (hipHostMalloc((void **)&d->trip_host, sizeof(int32_t), hipHostMallocMapped) != hipSuccess) return;
    *d->trip_host = 0;
    if (hipHostGetDevicePointer((void **)&d->trip_dev, d->trip_host, 0) != hipSuccess) {
        (void)hipHostFree(d->trip_host);
        d->trip_host = nullptr;
        return;
    }
    d->xcd_grouped.store(true);
}
struct fhip_stream {
    fhip_device *dev;
    hipStream_t s;
};
struct fhip_event {
    fhip_device *dev;
    hipEvent_t e;
};
struct fhip_graph {
    fhip_device *dev;
    hipGraph_t graph;
    hipGraphExec_t exec;
};

namespace fhip {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int hip_fail(hipError_t e, const char *what) {
    set_error("HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
    return FHIP_ERR_HIP;
}

static int elem_bytes(fhip_dtype d) { return d == FHIP_F32 ? 4 : 2; }

static bool dtype_ok(int d) { return d == FHIP_F32 || d == FHIP_F16 || d == FHIP_BF16; }

// ---- validation (host only) -------------------------------------------------------------------

static int validate(const fhip_attn_args *a) {
    if (!a) {
        set_error("args is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    if (!dtype_ok(a->dtype) || !dtype_ok(a->out_dtype)) {
        set_error("unknown dtype %d / out_dtype %d", (int)a->dtype, (int)a->out_dtype);
        return FHIP_ERR_INVALID_ARG;
    }
    if (a->out_dtype != a->dtype && !(a->out_dtype == FHIP_F32 && a->dtype != FHIP_F32)) {
        set_error("out_dtype must equal dtype, or be f32 for 16-bit inputs");
        return FHIP_ERR_INVALID_ARG;
    }
    const uint32_t *qs = a->q.shape, *ks = a->k.shape, *vs = a->v.shape, *os = a->out.shape;
    for (int i = 0; i < 4; i++) {
        if (qs[i] > 0x7fffffffu || ks[i] > 0x7fffffffu) {
            set_error("dimension larger than 2^31-1");
            return FHIP_ERR_INVALID_ARG;
        }
    }
    const uint32_t B = qs[0], H = qs[1], Sq = qs[2], D = qs[3];
    const uint32_t Hkv = ks[1], Skv = ks[2];
    // reference: assert!(num_heads.is_multiple_of(num_kv_heads), ...) flash_attention.rs:94-99
    // (u32::is_multiple_of(0) holds for 0 only)
    if (Hkv == 0 ? H != 0 : H % Hkv != 0) {
        set_error("Number of Q heads (%u) must be divisible by number of K/V heads (%u)", H, Hkv);
        return FHIP_ERR_INVALID_ARG;
    }
    if (ks[0] != B || ks[3] != D) {
        set_error("K shape [%u, %u, %u, %u] does not match Q shape [%u, %u, %u, %u] in batch/head_dim", ks[0],
                  ks[1], ks[2], ks[3], B, H, Sq, D);
        return FHIP_ERR_INVALID_ARG;
    }
    for (int i = 0; i < 4; i++)
        if (vs[i] != ks[i]) {
            set_error("V shape [%u, %u, %u, %u] does not match K shape [%u, %u, %u, %u]", vs[0], vs[1], vs[2],
                      vs[3], ks[0], ks[1], ks[2], ks[3]);
            return FHIP_ERR_INVALID_ARG;
        }
    for (int i = 0; i < 4; i++)
        if (os[i] != qs[i]) {
            set_error("output shape [%u, %u, %u, %u] does not match Q shape [%u, %u, %u, %u]", os[0], os[1],
                      os[2], os[3], B, H, Sq, D);
            return FHIP_ERR_INVALID_ARG;
        }
    // a tensor without elements needs no memory
    const bool q_empty = B == 0 || H == 0 || Sq == 0 || D == 0, kv_empty = B == 0 || Hkv == 0 || Skv == 0 || D == 0;
    if ((!q_empty && (!a->q.ptr || !a->out.ptr)) || (!kv_empty && (!a->k.ptr || !a->v.ptr))) {
        set_error("q, k, v and out need device pointers");
        return FHIP_ERR_INVALID_ARG;
    }
    for (int i = 0; i < 4 && !q_empty; i++)
        if (os[i] > 1 && a->out.stride[i] == 0) {
            set_error("output stride %d is 0 (overlapping writes)", i);
            return FHIP_ERR_INVALID_ARG;
        }
    if (a->mask_intervals && (a->mask_kind == FHIP_MASK_NONE || ((uintptr_t)a->mask_intervals & 15) != 0)) {
        set_error("mask_intervals needs a mask tensor and a 16-byte aligned table");
        return FHIP_ERR_INVALID_ARG;
    }
    if (!std::isfinite(a->scale)) {
        set_error("scale must be finite");
        return FHIP_ERR_INVALID_ARG;
    }
    switch (a->mask_kind) {
        case FHIP_MASK_NONE:
            if (a->mask.ptr) {
                set_error("mask pointer given with FHIP_MASK_NONE");
                return FHIP_ERR_INVALID_ARG;
            }
            break;
        case FHIP_MASK_QK:
            // reference: assert_eq!(m_shape, [q_seq_len, kv_seq_len], ...) flash_attention.rs:153-160
            if (a->mask.shape[0] != Sq || a->mask.shape[1] != Skv) {
                set_error("QKMask shape [%u, %u] does not match expected [%u, %u]", a->mask.shape[0],
                          a->mask.shape[1], Sq, Skv);
                return FHIP_ERR_INVALID_ARG;
            }
            break;
        case FHIP_MASK_BATCH_KEY:
            // reference: flash_attention.rs:165-172
            if (a->mask.shape[0] != B || a->mask.shape[1] != Skv) {
                set_error("BatchKeyMask shape [%u, %u] does not match expected [%u, %u]", a->mask.shape[0],
                          a->mask.shape[1], B, Skv);
                return FHIP_ERR_INVALID_ARG;
            }
            break;
        default:
            set_error("unknown mask_kind %d", (int)a->mask_kind);
            return FHIP_ERR_INVALID_ARG;
    }
    if (a->mask_kind != FHIP_MASK_NONE && !a->mask.ptr) {
        set_error("mask_kind set but mask pointer is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    if (a->analytic.enabled) {
        if (a->mask_kind != FHIP_MASK_NONE) {
            set_error("analytic mask and mask tensor are mutually exclusive");
            return FHIP_ERR_INVALID_ARG;
        }
        if (a->analytic.window < 0 || a->analytic.q_pos_offset < 0) {
            set_error("analytic mask: window and q_pos_offset must be >= 0");
            return FHIP_ERR_INVALID_ARG;
        }
    }
    if (D > 512) {
        set_error("head_dim %u > 512 has no kernel", D);
        return FHIP_ERR_UNSUPPORTED;
    }
    return FHIP_OK;
}

// Calls whose result is fixed by the shapes alone.  No output element: nothing to do.  No key (Skv == 0)
// but output elements: the reference's composite multiplies a [Sq, 0] matrix of probabilities with a
// [0, D] matrix of values, which is all zeros (fusor flash_attention.rs:141-199: the softmax of an empty
// row is empty, no 0/0 is ever formed).
static bool output_is_empty(const fhip_attn_args *a) {
    return a->q.shape[0] == 0 || a->q.shape[1] == 0 || a->q.shape[2] == 0 || a->q.shape[3] == 0;
}
static bool no_keys(const fhip_attn_args *a) { return a->k.shape[2] == 0; }

// rows readable in pieces of `bytes` (16, or 8 for the four-element pieces of a 16-bit row)
static bool rows_vectorizable(const fhip_tensor4 &t, int eb, int bytes = 16) {
    const int per = bytes / eb;
    if (t.shape[3] > 1 && t.stride[3] != 1) return false;
    if ((((uintptr_t)t.ptr + t.offset * (uint64_t)eb) & (uintptr_t)(bytes - 1)) != 0) return false;
    for (int i = 0; i < 3; i++)
        if (t.shape[i] > 1 && (t.stride[i] % per) != 0) return false;
    return true;
}

// Query rows per sequence the split-KV decode kernels take: the single row of a decode step, and the few rows of a
// multi-token step (a draft being verified, a short piece of a prompt), which ride as further columns beside the
// query heads that share a KV head.
constexpr uint32_t DECODE_MAX_ROWS = 4;

static bool decode_eligible(const fhip_attn_args *a) {
    const uint32_t D = a->q.shape[3], rows = a->q.shape[2];
    if (rows < 1) return false;
    if (rows > DECODE_MAX_ROWS) {
        // more rows (a longer draft, a short piece of a prompt) still ride along while rows x group fit the columns one
        // workgroup of a matrix-core variant takes: two blocks of 16 up to head_dim 128, one above
        const uint32_t Hkv = a->k.shape[1], G = Hkv ? a->q.shape[1] / Hkv : 0;
        const bool matrix_variant = D % 32 == 0 && D >= 32 && D <= 256u;
        // f32: two column blocks per workgroup up to head_dim 192, and two workgroups per KV head (each streams the
        // cache) still beat the f32 prefill kernel
        const uint32_t max_cols = a->dtype == FHIP_F32 ? (D <= 192 ? 64u : 32u) : (D <= 128 ? 32u : 16u);
        if (!matrix_variant || G == 0 || rows * G > max_cols) return false;
    }
    if (D % 8 != 0 || D < 8 || D > 256) return false;
    const int eb = a->dtype == FHIP_F32 ? 4 : 2;
    if (!rows_vectorizable(a->k, eb) || !rows_vectorizable(a->v, eb)) return false;
    if (a->k.stride[2] < 0 || a->v.stride[2] < 0) return false;
    return true;
}

static bool prefill_mfma_eligible(const fhip_attn_args *a) {
    if (a->dtype == FHIP_F32) return false;
    const uint32_t D = a->q.shape[3];
    // 64 / 96 / 128: attn_prefill_mfma.hip; every other multiple of 8 up to 256 (padded to the next multiple of 32):
    // attn_prefill_mfma_wide.hip
    const bool wide = !(D == 64 || D == 96 || D == 128);
    if (D % 8 != 0 || D < 8 || D > 256) return false;
    if (!rows_vectorizable(a->q, 2) || !rows_vectorizable(a->k, 2) || !rows_vectorizable(a->v, 2)) return false;
    // the kernel for 64 / 96 / 128 multiplies Q by the power-of-two part of scale * log2(e): that power must be at most
    // 1 so that no finite element can leave the type's range (the wide-head kernel scales the scores in f32 only)
    if (!wide && (!(a->scale > 0.0f) || !(a->scale * 1.4426950408889634f < 2.0f))) return false;
    // K/V rows are fetched through 32-bit buffer offsets: rows must not overlap and one (batch, kv
    // head) slice must span less than 2 GiB
    const uint64_t Skv = a->k.shape[2];
    if (a->k.stride[2] < (int64_t)D || a->v.stride[2] < (int64_t)D) return false;
    if (Skv * (uint64_t)a->k.stride[2] * 2 >= 0x7fffffffull || Skv * (uint64_t)a->v.stride[2] * 2 >= 0x7fffffffull)
        return false;
    return true;
}

// The tiled kernel that computes in f32 on the f32 matrix cores.  It is THE prefill kernel for f32 tensors and the
// second choice for 16-bit ones (rows widened on load): head dims and mask tensors their own kernel does not take.
static bool prefill_f32_eligible(const fhip_attn_args *a) {
    const uint32_t D = a->q.shape[3];
    if (D % 4 != 0 || D > 256) return false;  // rows are padded with zeros to the tile width on the way into LDS
    if (!(a->scale > 0.0f)) return false;
    const int eb = elem_bytes(a->dtype), piece = 4 * eb;  // rows are read four elements at a time
    if (!rows_vectorizable(a->q, eb, piece) || !rows_vectorizable(a->k, eb, piece) || !rows_vectorizable(a->v, eb, piece))
        return false;
    return true;
}

// what fhip_mask_intervals leaves in the first word of its table when some row of the mask is not an interval
constexpr int32_t MASK_TABLE_BAD = 1;

// A dense mask reaches the tiled prefill kernels in interval form (mask_intervals.hip), which needs
// device scratch: 16 bytes for the mark of a mask whose rows are not all intervals, then {lo, hi} per row.
static size_t mask_scratch_bytes(const fhip_attn_args *a) {
    if (a->mask_kind == FHIP_MASK_NONE || a->mask_intervals) return 0;  // no mask, or its interval form comes with the call
    return mask_intervals_bytes(a->mask_kind == FHIP_MASK_QK ? (int)a->q.shape[2] : (int)a->q.shape[0]);
}
static bool mask_scratch_ok(const fhip_attn_args *a, bool assume_workspace) {
    if (a->mask_kind == FHIP_MASK_NONE || assume_workspace || a->mask_intervals) return true;
    return a->workspace && ((uintptr_t)a->workspace & 15) == 0 && a->workspace_bytes >= mask_scratch_bytes(a);
}

// The f32 tiled kernel can add a mask tensor element by element (no scratch, no interval form) up to head_dim 128.
static bool f32_adds_masks(const fhip_attn_args *a) { return a->q.shape[3] <= 128; }

// At head_dim <= 64 the f32 tiled kernel holds both mask forms: it reads what the scan found and no hand-over kernel
// is queued behind it.
static bool f32_serves_both_mask_forms(const fhip_attn_args *a) { return a->q.shape[3] <= 64; }

// The keys a decode call can see at all, when the analytic descriptor alone says so (no mask tensor, no per-sequence key
// counts): [*lo0, *lo0 + *len) with *lo0 a multiple of 128.  The kernels are handed the tensors from key *lo0 on (and the
// query position moved by as much), so the split-KV plan covers this range only: a window of 4096 keys at the end of a
// 16384-key cache is spread over as many workgroups as a 4096-key cache would be.
static void decode_visible_range(const fhip_attn_args *a, int *lo0, int *len) {
    const int64_t Skv = a->k.shape[2], rows = a->q.shape[2];
    int64_t lo = 0, hi = Skv;
    if (a->analytic.enabled && !a->kv_lens && a->mask_kind == FHIP_MASK_NONE) {
        if (a->analytic.causal) hi = std::min<int64_t>(hi, a->analytic.q_pos_offset + rows);
        if (a->analytic.window > 0) lo = std::max<int64_t>(0, a->analytic.q_pos_offset - a->analytic.window + 1);
    }
    if (hi <= lo) lo = 0, hi = Skv;  // nothing visible: the rows come out NaN however the keys are split
    *lo0 = (int)(lo / 128 * 128);
    *len = (int)(hi - *lo0);
}

// Key split of a call the f32-arithmetic tiled kernel serves (few query rows on a long cache), and where its
// partial results go in the workspace: behind the mask scratch, 256-byte aligned.
static void f32_split_plan(const fhip_attn_args *a, int cus, int *nsplit, int *chunk) {
    const bool causal_square = a->analytic.enabled && a->analytic.causal && 2ull * a->q.shape[2] > a->k.shape[2];
    const int Hkv = (int)a->k.shape[1];
    prefill_f32_plan((int)a->q.shape[0], (int)a->q.shape[1], Hkv ? (int)a->q.shape[1] / Hkv : 1, (int)a->q.shape[2],
                     (int)a->k.shape[2], (int)a->q.shape[3], causal_square, cus > 0 ? cus : 256, nsplit, chunk);
}
static size_t f32_partials_offset(const fhip_attn_args *a) { return (mask_scratch_bytes(a) + 255) & ~(size_t)255; }
static void mfma_split_plan(const fhip_attn_args *a, int cus, int *nsplit, int *chunk) {
    if (a->force_kernel == FHIP_KERNEL_PREFILL_MFMA_ROWS64) {  // that form never splits the keys
        *nsplit = 1;
        *chunk = (int)a->k.shape[2];
        return;
    }
    const bool causal_square = a->analytic.enabled && a->analytic.causal && 2ull * a->q.shape[2] > a->k.shape[2];
    const int Hkv = (int)a->k.shape[1];
    if (!(a->q.shape[3] == 64 || a->q.shape[3] == 96 || a->q.shape[3] == 128))  // the wide-head form: 128-row query blocks
        prefill_mfma_wide_plan((int)a->q.shape[0], (int)a->q.shape[1], Hkv ? (int)a->q.shape[1] / Hkv : 1, (int)a->q.shape[2],
                               (int)a->k.shape[2], causal_square, cus > 0 ? cus : 256, nsplit, chunk);
    else
        prefill_mfma_plan((int)a->q.shape[0], (int)a->q.shape[1], Hkv ? (int)a->q.shape[1] / Hkv : 1, (int)a->q.shape[2],
                          (int)a->k.shape[2], causal_square, cus > 0 ? cus : 256, nsplit, chunk);
}

// A workspace too small for the planned key split still takes the largest split that fits (shares stay multiples of 64
// keys, which every tiled kernel's tile size divides); below two shares the call runs unsplit.
static void fit_split(int Skv, size_t bytes_per_share, size_t avail, int *nsplit, int *chunk) {
    if (*nsplit <= 1 || bytes_per_share == 0 || bytes_per_share * (size_t)*nsplit <= avail) return;
    const long fit = (long)(avail / bytes_per_share);
    long c = fit >= 2 ? ((long)Skv + fit - 1) / fit : Skv;
    c = (c + 63) / 64 * 64;
    *chunk = (int)c;
    *nsplit = (int)((Skv + c - 1) / c);
    if (*nsplit <= 1) *nsplit = 1, *chunk = Skv;
}

// assume_workspace: answer as if the caller had provided the scratch a masked tiled call needs
// (the size query); otherwise a masked call without enough scratch takes the general kernel.
static int select_kernel(const fhip_attn_args *a, int32_t *id, bool assume_workspace = false) {
    const int f = a->force_kernel;
    if (output_is_empty(a) || no_keys(a)) {  // answered without an attention kernel
        *id = FHIP_KERNEL_GENERIC;
        return FHIP_OK;
    }
    const bool mask_ok = mask_scratch_ok(a, assume_workspace);
    if (f != FHIP_KERNEL_AUTO) {
        bool ok = false;
        switch (f) {
            case FHIP_KERNEL_GENERIC: ok = true; break;
            case FHIP_KERNEL_PREFILL_MFMA: ok = prefill_mfma_eligible(a) && mask_ok; break;
            case FHIP_KERNEL_PREFILL_MFMA_ROWS64:
                ok = prefill_mfma_eligible(a) && mask_ok && prefill_mfma_rows64_takes((int)a->q.shape[3], a->scale);
                break;
            case FHIP_KERNEL_PREFILL_F32: ok = prefill_f32_eligible(a) && (mask_ok || f32_adds_masks(a)); break;
            case FHIP_KERNEL_DECODE_SPLITKV: ok = decode_eligible(a); break;
            default: set_error("unknown force_kernel %d", f); return FHIP_ERR_INVALID_ARG;
        }
        if (!ok) {
            set_error("force_kernel %d cannot run these arguments (dtype/head_dim/stride constraints, or a mask without "
                      "the workspace its interval form needs)", f);
            return FHIP_ERR_UNSUPPORTED;
        }
        // (the forced form of the tiled 16-bit kernel is that kernel to everything that follows; AttnParams carries the form)
        *id = f == FHIP_KERNEL_PREFILL_MFMA_ROWS64 ? (int)FHIP_KERNEL_PREFILL_MFMA : f;
        return FHIP_OK;
    }
    if (decode_eligible(a))
        *id = FHIP_KERNEL_DECODE_SPLITKV;
    else if (prefill_mfma_eligible(a) && mask_ok)
        *id = FHIP_KERNEL_PREFILL_MFMA;
    else if (prefill_f32_eligible(a) && (mask_ok || f32_adds_masks(a)))
        *id = FHIP_KERNEL_PREFILL_F32;
    else
        *id = FHIP_KERNEL_GENERIC;
    return FHIP_OK;
}

static void fill_params(const fhip_attn_args *a, AttnParams *p) {
    const int eb = elem_bytes(a->dtype);
    const int ob = elem_bytes(a->out_dtype);
    memset(p, 0, sizeof(*p));
    p->q = (const char *)a->q.ptr + a->q.offset * eb;
    p->k = (const char *)a->k.ptr + a->k.offset * eb;
    p->v = (const char *)a->v.ptr + a->v.offset * eb;
    p->out = (char *)a->out.ptr + a->out.offset * ob;
    for (int i = 0; i < 4; i++) {
        p->qs[i] = a->q.stride[i];
        p->ks[i] = a->k.stride[i];
        p->vs[i] = a->v.stride[i];
        p->os[i] = a->out.stride[i];
    }
    p->B = (int)a->q.shape[0];
    p->H = (int)a->q.shape[1];
    p->Sq = (int)a->q.shape[2];
    p->D = (int)a->q.shape[3];
    p->Hkv = (int)a->k.shape[1];
    p->Skv = (int)a->k.shape[2];
    p->G = p->H / p->Hkv;
    p->mask_kind = a->mask_kind;
    if (a->mask_kind != FHIP_MASK_NONE) {
        p->mask = (const char *)a->mask.ptr + a->mask.offset * eb;
        p->ms0 = a->mask.stride[0];
        p->ms1 = a->mask.stride[1];
    }
    p->analytic = a->analytic.enabled ? 1 : 0;
    p->causal = a->analytic.enabled ? (a->analytic.causal ? 1 : 0) : 0;
    p->q_pos_offset = a->analytic.q_pos_offset;
    p->window = a->analytic.enabled ? a->analytic.window : 0;
    p->kv_lens = a->kv_lens;
    p->scale = a->scale;
    p->out_f32 = (a->out_dtype == FHIP_F32 && a->dtype != FHIP_F32) ? 1 : 0;
}

}  // namespace fhip

using namespace fhip;

extern "C" {

const char *fhip_last_error(void) { return g_err; }

const char *fhip_version(void) { return "fusor-hip 0.1 (gfx950)"; }

int fhip_device_count(int32_t *count) {
    if (!count) {
        set_error("count is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        *count = 0;
        return hip_fail(e, "hipGetDeviceCount");
    }
    *count = n;
    return FHIP_OK;
}

int fhip_device_create(int32_t ordinal, fhip_device **out) {
    if (!out) {
        set_error("out is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    *out = nullptr;
    int n = 0;
    FHIP_HIP_CHECK(hipGetDeviceCount(&n));
    if (ordinal < 0 || ordinal >= n) {
        set_error("device ordinal %d out of range (%d devices)", ordinal, n);
        return FHIP_ERR_INVALID_ARG;
    }
    fhip_device *d = new (std::nothrow) fhip_device();
    if (!d) {
        set_error("out of host memory");
        return FHIP_ERR_HIP;
    }
    d->ordinal = ordinal;
    // handles of one device start their marks far apart, so that two of them sharing a workspace do not collide
    d->next_tag.store(0x5eed0001u + (uint32_t)((uintptr_t)d >> 4) * 2654435761u, std::memory_order_relaxed);
    hipError_t e = hipGetDeviceProperties(&d->prop, ordinal);
    if (e != hipSuccess) {
        delete d;
        return hip_fail(e, "hipGetDeviceProperties");
    }
    if (strncmp(d->prop.gcnArchName, "gfx950", 6) != 0) {
        set_error("device %d is %s; this library carries gfx950 code only", ordinal, d->prop.gcnArchName);
        delete d;
        return FHIP_ERR_UNSUPPORTED;
    }
    // this device's copy of the static workspace (the lookup is per device: it must be the current one)
    // (the calling thread's current device is put back afterwards)
    d->scratch_ptr = nullptr;
    int previous = -1;
    (void)hipGetDevice(&previous);
    e = hipSetDevice(ordinal);
    if (e == hipSuccess) e = hipGetSymbolAddress((void **)&d->scratch_ptr, HIP_SYMBOL(scratch));
    if (e == hipSuccess && d->scratch_ptr) probe_xcd_grouping(d);
    if (previous >= 0 && previous != ordinal) (void)hipSetDevice(previous);
    if (e != hipSuccess || !d->scratch_ptr) {
        delete d;
        return hip_fail(e, "hipGetSymbolAddress(scratch)");
    }
    *out = d;
    return FHIP_OK;
}

int fhip_device_destroy(fhip_device *dev) {
    if (dev && dev->trip_host) (void)hipHostFree(dev->trip_host);
    delete dev;
    return FHIP_OK;
}

int fhip_device_get_info(fhip_device *dev, fhip_device_info *info) {
    if (!dev || !info) {
        set_error("dev/info is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    memset(info, 0, sizeof(*info));
    snprintf(info->name, sizeof(info->name), "%s", dev->prop.name);
    snprintf(info->arch, sizeof(info->arch), "%s", dev->prop.gcnArchName);
    info->compute_units = dev->prop.multiProcessorCount;
    info->wavefront_size = dev->prop.warpSize;
    info->clock_khz = dev->prop.clockRate;
    info->memory_clock_khz = dev->prop.memoryClockRate;
    info->memory_bus_bits = dev->prop.memoryBusWidth;
    info->total_memory = dev->prop.totalGlobalMem;
    info->lds_per_cu = dev->prop.maxSharedMemoryPerMultiProcessor;
    info->l2_bytes = (uint64_t)dev->prop.l2CacheSize;
    return FHIP_OK;
}

int fhip_stream_create(fhip_device *dev, fhip_stream **out) {
    if (!dev || !out) {
        set_error("dev/out is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    *out = nullptr;
    FHIP_HIP_CHECK(hipSetDevice(dev->ordinal));
    hipStream_t s;
    FHIP_HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    fhip_stream *st = new (std::nothrow) fhip_stream();
    if (!st) {
        (void)hipStreamDestroy(s);
        set_error("out of host memory");
        return FHIP_ERR_HIP;
    }
    st->dev = dev;
    st->s = s;
    *out = st;
    return FHIP_OK;
}

int fhip_stream_destroy(fhip_stream *s) {
    if (!s) return FHIP_OK;
    hipError_t e = hipStreamDestroy(s->s);
    delete s;
    if (e != hipSuccess) return hip_fail(e, "hipStreamDestroy");
    return FHIP_OK;
}

int fhip_stream_synchronize(fhip_stream *s) {
    if (!s) {
        set_error("stream is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    FHIP_HIP_CHECK(hipStreamSynchronize(s->s));
    return FHIP_OK;
}

int fhip_malloc(fhip_device *dev, size_t bytes, void **out) {
    if (!dev || !out) {
        set_error("dev/out is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    *out = nullptr;
    FHIP_HIP_CHECK(hipSetDevice(dev->ordinal));
    FHIP_HIP_CHECK(hipMalloc(out, bytes ? bytes : 1));
    return FHIP_OK;
}

int fhip_free(fhip_device *dev, void *ptr) {
    if (!dev) {
        set_error("dev is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    if (!ptr) return FHIP_OK;
    FHIP_HIP_CHECK(hipSetDevice(dev->ordinal));
    FHIP_HIP_CHECK(hipFree(ptr));
    return FHIP_OK;
}

int fhip_memcpy_h2d(fhip_stream *s, void *dst, const void *src, size_t bytes) {
    if (!s || (bytes && (!dst || !src))) {
        set_error("memcpy_h2d: NULL argument");
        return FHIP_ERR_INVALID_ARG;
    }
    if (!bytes) return FHIP_OK;
    // pageable host memory: the copy is staged by the runtime, the host buffer is reusable on return
    FHIP_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, s->s));
    FHIP_HIP_CHECK(hipStreamSynchronize(s->s));
    return FHIP_OK;
}

int fhip_memcpy_d2h(fhip_stream *s, void *dst, const void *src, size_t bytes) {
    if (!s || (bytes && (!dst || !src))) {
        set_error("memcpy_d2h: NULL argument");
        return FHIP_ERR_INVALID_ARG;
    }
    if (!bytes) return FHIP_OK;
    FHIP_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s->s));
    FHIP_HIP_CHECK(hipStreamSynchronize(s->s));
    return FHIP_OK;
}

int fhip_memcpy_d2d(fhip_stream *s, void *dst, const void *src, size_t bytes) {
    if (!s || (bytes && (!dst || !src))) {
        set_error("memcpy_d2d: NULL argument");
        return FHIP_ERR_INVALID_ARG;
    }
    if (!bytes) return FHIP_OK;
    FHIP_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, s->s));
    return FHIP_OK;
}

int fhip_memset(fhip_stream *s, void *dst, int value, size_t bytes) {
    if (!s || (bytes && !dst)) {
        set_error("memset: NULL argument");
        return FHIP_ERR_INVALID_ARG;
    }
    if (!bytes) return FHIP_OK;
    FHIP_HIP_CHECK(hipSetDevice(s->dev->ordinal));
    return launch_fill_bytes(dst, value, bytes, s->s);  // a kernel, not a memset node: safe to record into a graph
}

// ---- stream capture: a sequence of calls recorded once and replayed with one launch --------------------

int fhip_stream_begin_capture(fhip_stream *s) {
    if (!s) {
        set_error("stream is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    FHIP_HIP_CHECK(hipSetDevice(s->dev->ordinal));
    FHIP_HIP_CHECK(hipStreamBeginCapture(s->s, hipStreamCaptureModeThreadLocal));
    return FHIP_OK;
}

int fhip_stream_end_capture(fhip_stream *s, fhip_graph **out) {
    if (!s || !out) {
        set_error("stream/out is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    *out = nullptr;
    hipGraph_t g = nullptr;
    FHIP_HIP_CHECK(hipStreamEndCapture(s->s, &g));
    if (!g) {
        set_error("the capture produced no graph (a call in it failed)");
        return FHIP_ERR_HIP;
    }
    hipGraphExec_t ex = nullptr;
    hipError_t e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(g);
        return hip_fail(e, "hipGraphInstantiate");
    }
    fhip_graph *gr = new (std::nothrow) fhip_graph();
    if (!gr) {
        (void)hipGraphExecDestroy(ex);
        (void)hipGraphDestroy(g);
        set_error("out of host memory");
        return FHIP_ERR_HIP;
    }
    gr->dev = s->dev;
    gr->graph = g;
    gr->exec = ex;
    *out = gr;
    return FHIP_OK;
}

int fhip_graph_launch(fhip_graph *g, fhip_stream *s) {
    if (!g || !s) {
        set_error("graph/stream is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    FHIP_HIP_CHECK(hipSetDevice(s->dev->ordinal));
    FHIP_HIP_CHECK(hipGraphLaunch(g->exec, s->s));
    return FHIP_OK;
}

int fhip_graph_destroy(fhip_graph *g) {
    if (!g) return FHIP_OK;
    hipError_t e1 = hipGraphExecDestroy(g->exec), e2 = hipGraphDestroy(g->graph);
    delete g;
    if (e1 != hipSuccess) return hip_fail(e1, "hipGraphExecDestroy");
    if (e2 != hipSuccess) return hip_fail(e2, "hipGraphDestroy");
    return FHIP_OK;
}

int fhip_event_create(fhip_device *dev, fhip_event **out) {
    if (!dev || !out) {
        set_error("dev/out is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    *out = nullptr;
    FHIP_HIP_CHECK(hipSetDevice(dev->ordinal));
    hipEvent_t e;
    FHIP_HIP_CHECK(hipEventCreate(&e));
    fhip_event *ev = new (std::nothrow) fhip_event();
    if (!ev) {
        (void)hipEventDestroy(e);
        set_error("out of host memory");
        return FHIP_ERR_HIP;
    }
    ev->dev = dev;
    ev->e = e;
    *out = ev;
    return FHIP_OK;
}

int fhip_event_destroy(fhip_event *e) {
    if (!e) return FHIP_OK;
    hipError_t r = hipEventDestroy(e->e);
    delete e;
    if (r != hipSuccess) return hip_fail(r, "hipEventDestroy");
    return FHIP_OK;
}

int fhip_event_record(fhip_event *e, fhip_stream *s) {
    if (!e || !s) {
        set_error("event/stream is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    FHIP_HIP_CHECK(hipEventRecord(e->e, s->s));
    return FHIP_OK;
}

int fhip_event_synchronize(fhip_event *e) {
    if (!e) {
        set_error("event is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    FHIP_HIP_CHECK(hipEventSynchronize(e->e));
    return FHIP_OK;
}

int fhip_event_elapsed_ms(fhip_event *start, fhip_event *stop, float *ms) {
    if (!start || !stop || !ms) {
        set_error("event_elapsed_ms: NULL argument");
        return FHIP_ERR_INVALID_ARG;
    }
    FHIP_HIP_CHECK(hipEventElapsedTime(ms, start->e, stop->e));
    return FHIP_OK;
}

// ---- attention ----------------------------------------------------------------------------------

int fhip_flash_attention_validate(const fhip_attn_args *args) { return validate(args); }

int fhip_flash_attention_select(const fhip_attn_args *args, int32_t *kernel_id) {
    if (!kernel_id) {
        set_error("kernel_id is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    int rc = validate(args);
    if (rc) return rc;
    rc = select_kernel(args, kernel_id);
    if (rc == FHIP_OK && args->force_kernel == FHIP_KERNEL_PREFILL_MFMA_ROWS64 && *kernel_id == FHIP_KERNEL_PREFILL_MFMA)
        *kernel_id = FHIP_KERNEL_PREFILL_MFMA_ROWS64;
    return rc;
}

int fhip_flash_attention_workspace_bytes(const fhip_attn_args *args, int32_t compute_units, size_t *bytes) {
    if (!bytes) {
        set_error("bytes is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    *bytes = 0;
    int rc = validate(args);
    if (rc) return rc;
    int32_t id;
    rc = select_kernel(args, &id, true);
    if (rc) return rc;
    if (output_is_empty(args) || no_keys(args)) return FHIP_OK;
    if (id == FHIP_KERNEL_PREFILL_MFMA || id == FHIP_KERNEL_PREFILL_F32) *bytes = mask_scratch_bytes(args);
    if (id == FHIP_KERNEL_PREFILL_F32) {
        int ns, chunk;
        f32_split_plan(args, compute_units, &ns, &chunk);
        const size_t part = prefill_f32_workspace_bytes((int)args->q.shape[0], (int)args->q.shape[1], (int)args->q.shape[2],
                                                        (int)args->q.shape[3], ns);
        if (part) *bytes = f32_partials_offset(args) + part;
    }
    if (id == FHIP_KERNEL_PREFILL_MFMA) {
        int ns, chunk;
        mfma_split_plan(args, compute_units, &ns, &chunk);
        const size_t part = prefill_mfma_workspace_bytes((int)args->q.shape[0], (int)args->q.shape[1], (int)args->q.shape[2],
                                                         (int)args->q.shape[3], ns);
        if (part) *bytes = f32_partials_offset(args) + part;
    }
    if (id == FHIP_KERNEL_DECODE_SPLITKV) {
        int chunk, nsplit, waves;
        const int B = (int)args->q.shape[0], H = (int)args->q.shape[1], D = (int)args->q.shape[3];
        const int Hkv = (int)args->k.shape[1], Skv = (int)args->k.shape[2], rows = (int)args->q.shape[2];
        int lo0, len;
        decode_visible_range(args, &lo0, &len);
        (void)Skv;
        decode_plan(B, Hkv, H / Hkv * rows, len, D, compute_units > 0 ? compute_units : 256, args->kv_lens != nullptr,
                    args->dtype == FHIP_F32, &chunk, &nsplit, &waves);
        *bytes = decode_workspace_bytes(B, H * rows, Hkv, D, nsplit);
    }
    return FHIP_OK;
}

// The plan of a split-KV decode call: the visible stretch of the cache, the split, and whether the splits are merged
// inside the main kernel (when the device's workgroups are grouped by XCD as that form needs, see probe_xcd_grouping).
static void plan_decode_call(fhip_device *dev, const fhip_attn_args *args, AttnParams *p) {
    int lo0, vis_len;
    decode_visible_range(args, &lo0, &vis_len);
    if (lo0 > 0 || vis_len < p->Skv) {  // the kernels see keys lo0 .. lo0 + vis_len as keys 0 .. vis_len
        const int64_t eb = elem_bytes(args->dtype);
        p->k = (const char *)p->k + lo0 * p->ks[2] * eb;
        p->v = (const char *)p->v + lo0 * p->vs[2] * eb;
        p->Skv = vis_len;
        p->q_pos_offset -= lo0;
    }
    decode_plan(p->B, p->Hkv, p->G * p->Sq, p->Skv, p->D, dev->prop.multiProcessorCount, p->kv_lens != nullptr,
                args->dtype == FHIP_F32, &p->chunk, &p->nsplit, &p->dec_waves);
    int stride;
    size_t ctr_off;
    p->dec_fused = 0;
    if (dev->xcd_grouped.load() && decode_fused_layout(*p, args->dtype == FHIP_F32, &stride, &ctr_off)) {
        p->dec_fused = 1;
        p->dec_unit_stride = stride;
        p->dec_counters_offset = ctr_off;
    }
}

// the 16-bit tiled prefill kernels: 64 / 96 / 128, and the wide-head form above
static int launch_mfma_by_head_dim(const AttnParams &p, fhip_dtype dtype, hipStream_t stream) {
    // the form of four wavefronts with 64 rows each (attn_prefill_mfma_rows64.hip), when the caller forces it: measured
    // 1-3 % slower than the 256-row form of eight wavefronts on the benchmark prompts (fewer LDS reads and a higher clock,
    // but a lone wavefront per SIMD issues everything in order), so it is never chosen
    if (p.pf_rows64) return launch_prefill_mfma_rows64(p, dtype, stream);
    return (p.D == 64 || p.D == 96 || p.D == 128) ? launch_prefill_mfma(p, dtype, stream) : launch_prefill_mfma_wide(p, dtype, stream);
}

int fhip_flash_attention_decode_plan(fhip_stream *s, const fhip_attn_args *args, fhip_decode_plan_info *info) {
    if (!s || !info) {
        set_error("stream/info is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    memset(info, 0, sizeof(*info));
    int rc = validate(args);
    if (rc) return rc;
    int32_t id;
    rc = select_kernel(args, &id);
    if (rc) return rc;
    if (id != FHIP_KERNEL_DECODE_SPLITKV || output_is_empty(args) || no_keys(args)) return FHIP_OK;
    AttnParams p;
    fill_params(args, &p);
    plan_decode_call(s->dev, args, &p);
    info->is_decode = 1;
    info->nsplit = p.nsplit;
    info->chunk = p.chunk;
    info->wavefronts = p.dec_waves;
    info->kernels = p.nsplit > 1 && !p.dec_fused ? 2 : 1;
    return FHIP_OK;
}

int fhip_flash_attention(fhip_stream *s, const fhip_attn_args *args) {
    if (!s) {
        set_error("stream is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    int rc = validate(args);
    if (rc) return rc;
    int32_t id;
    rc = select_kernel(args, &id);
    if (rc) return rc;
    FHIP_HIP_CHECK(hipSetDevice(s->dev->ordinal));
    if (output_is_empty(args) || no_keys(args)) {
        if (!output_is_empty(args)) {
            char *out = (char *)args->out.ptr + args->out.offset * (uint64_t)elem_bytes(args->out_dtype);
            rc = launch_fill_zero_rows(out, args->out.stride, args->out.shape, elem_bytes(args->out_dtype), s->s);
            if (rc) return rc;
        }
        // no attention kernel runs: the hooks still hold a valid (empty) interval
        if (args->main_kernel_start && args->main_kernel_done) FHIP_HIP_CHECK(hipEventRecord(args->main_kernel_start->e, s->s));
        if (args->main_kernel_done) FHIP_HIP_CHECK(hipEventRecord(args->main_kernel_done->e, s->s));
        return FHIP_OK;
    }
    AttnParams p;
    fill_params(args, &p);
    p.main_done = args->main_kernel_done ? args->main_kernel_done->e : nullptr;
    p.main_start = args->main_kernel_start && p.main_done ? args->main_kernel_start->e : nullptr;
    if (p.main_start) {
        // a dispatch that carries its own events cannot be recorded into a graph
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        FHIP_HIP_CHECK(hipStreamIsCapturing(s->s, &capturing));
        if (capturing != hipStreamCaptureStatusNone) {
            set_error("main_kernel_start cannot be used while the stream is being captured (use main_kernel_done alone)");
            return FHIP_ERR_UNSUPPORTED;
        }
    }
    p.cus = s->dev->prop.multiProcessorCount;
    if (id == FHIP_KERNEL_PREFILL_F32) {
        // few query rows on a long cache: split the keys over workgroups if the caller brought the scratch for it
        int ns, chunk;
        f32_split_plan(args, s->dev->prop.multiProcessorCount, &ns, &chunk);
        const size_t off = f32_partials_offset(args);
        const bool usable = args->workspace && ((uintptr_t)args->workspace & 15) == 0 && args->workspace_bytes > off;
        if (usable) fit_split(p.Skv, prefill_f32_workspace_bytes(p.B, p.H, p.Sq, p.D, 2) / 2, args->workspace_bytes - off, &ns, &chunk);
        const size_t part = prefill_f32_workspace_bytes(p.B, p.H, p.Sq, p.D, ns);
        if (part && usable && args->workspace_bytes >= off + part) {
            p.pf_nsplit = ns;
            p.pf_chunk = chunk;
            p.pf_pitch = p.D + 2;
            p.partials = (float *)((char *)args->workspace + off);
        }
    }
    if (id == FHIP_KERNEL_PREFILL_MFMA) {
        p.pf_rows64 = args->force_kernel == FHIP_KERNEL_PREFILL_MFMA_ROWS64;
        int ns, chunk;
        mfma_split_plan(args, s->dev->prop.multiProcessorCount, &ns, &chunk);
        const size_t off = f32_partials_offset(args);
        const bool usable = args->workspace && ((uintptr_t)args->workspace & 15) == 0 && args->workspace_bytes > off;
        if (usable) fit_split(p.Skv, prefill_mfma_workspace_bytes(p.B, p.H, p.Sq, p.D, 2) / 2, args->workspace_bytes - off, &ns, &chunk);
        const size_t part = prefill_mfma_workspace_bytes(p.B, p.H, p.Sq, p.D, ns);
        if (part && usable && args->workspace_bytes >= off + part) {
            p.pf_nsplit = ns;
            p.pf_chunk = chunk;
            p.pf_pitch = p.D + 4;  // rows of the partials are written in 16-byte pieces
            p.partials = (float *)((char *)args->workspace + off);
        }
    }
    if (id == FHIP_KERNEL_PREFILL_F32 && args->mask_kind != FHIP_MASK_NONE && !mask_scratch_ok(args, false)) {
        // no scratch for the interval form: the f32 kernel adds the mask tensor element by element
        rc = launch_prefill_f32(p, args->dtype, s->s);
        if (rc == FHIP_OK) FHIP_MARK_MAIN_DONE(p, s->s);
        return rc;
    }
    if ((id == FHIP_KERNEL_PREFILL_MFMA || id == FHIP_KERNEL_PREFILL_F32) && args->mask_kind != FHIP_MASK_NONE) {
        // dense mask: reduce it to one visible interval per row on the device; the tiled kernel skips the
        // masked tiles if every row is of that form.  If not, the f32-arithmetic kernel at head_dim <= 64 adds the
        // mask values itself; otherwise the kernel queued right behind the tiled one takes the call: the
        // f32-arithmetic kernel's mask-adding form (up to head_dim 128), else the general kernel.
        int32_t *bad = (int32_t *)args->workspace;
        int2 *iv = (int2 *)((char *)args->workspace + 16);
        if (args->mask_intervals) {
            // the interval form came with the call (fhip_mask_intervals, computed once for a mask that does not change):
            // no scan
            bad = (int32_t *)args->mask_intervals;
            iv = (int2 *)((char *)args->mask_intervals + 16);
            p.bad_tag = MASK_TABLE_BAD;
        } else {
            do p.bad_tag = (int32_t)s->dev->next_tag.fetch_add(1, std::memory_order_relaxed);
            while (p.bad_tag == 0);
            // A recorded call is replayed with the mark it was recorded with: a replay whose mask is not made of intervals
            // would leave that mark behind for every later replay.  Under capture the word is therefore cleared first
            // (by a kernel, which is what a graph may hold); an eager call's mark is new every time and needs no clearing.
            hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
            FHIP_HIP_CHECK(hipStreamIsCapturing(s->s, &capturing));
            if (capturing == hipStreamCaptureStatusActive) {
                rc = launch_fill_zero_bytes(bad, 16, s->s);
                if (rc) return rc;
            }
            rc = launch_mask_intervals(p, args->dtype, iv, bad, s->s);
            if (rc) return rc;
        }
        AttnParams pt = p;
        pt.iv = iv;
        pt.iv_bad = bad;
        const bool both_forms = id == FHIP_KERNEL_PREFILL_F32 && f32_serves_both_mask_forms(args);
        pt.iv_either = both_forms ? 1 : 0;
        rc = id == FHIP_KERNEL_PREFILL_MFMA ? launch_mfma_by_head_dim(pt, args->dtype, s->s) : launch_prefill_f32(pt, args->dtype, s->s);
        if (rc) return rc;
        FHIP_MARK_MAIN_DONE(p, s->s);
        if (both_forms) return FHIP_OK;
        AttnParams pg = p;
        pg.only_if_bad = bad;
        pg.main_start = pg.main_done = nullptr;  // the hook times the tiled kernel
        if (id == FHIP_KERNEL_PREFILL_MFMA) pg.pf_nsplit = 0;  // the split was planned for the other kernel's blocks
        return prefill_f32_eligible(args) && f32_adds_masks(args) ? launch_prefill_f32(pg, args->dtype, s->s)
                                                                  : launch_generic(pg, args->dtype, s->s);
    }
    switch (id) {
        case FHIP_KERNEL_GENERIC: rc = launch_generic(p, args->dtype, s->s); break;
        case FHIP_KERNEL_PREFILL_MFMA: rc = launch_mfma_by_head_dim(p, args->dtype, s->s); break;
        case FHIP_KERNEL_PREFILL_F32: rc = launch_prefill_f32(p, args->dtype, s->s); break;
        case FHIP_KERNEL_DECODE_SPLITKV: {
            plan_decode_call(s->dev, args, &p);
            const size_t need = decode_workspace_bytes(p.B, p.H * p.Sq, p.Hkv, p.D, p.nsplit);
            if (need > 0 && (!args->workspace || args->workspace_bytes < need)) {
                set_error("decode needs a workspace of %zu bytes, got %zu", need,
                          args->workspace ? args->workspace_bytes : (size_t)0);
                return FHIP_ERR_WORKSPACE;
            }
            if (need > 0) {
                if (((uintptr_t)args->workspace & 15) != 0) {
                    set_error("workspace must be 16-byte aligned");
                    return FHIP_ERR_WORKSPACE;
                }
                p.partials = (float *)args->workspace;
                fhip_device *dev = s->dev;
                if (dev->xcd_grouped.load() && *(volatile int32_t *)dev->trip_host != 0) {
                    dev->xcd_grouped.store(false);
                    set_error("the workgroups of one split-KV unit ran on different XCDs, which the device's probe had ruled out: "
                              "the result of an earlier decode call on this device may be wrong; later calls merge with a "
                              "second kernel");
                    return FHIP_ERR_HIP;
                }
                if (p.dec_fused) {
                    p.dec_counters = (uint32_t *)((char *)args->workspace + p.dec_counters_offset);
                    p.dec_trip = dev->trip_dev;
                    do p.dec_tag = dev->next_tag.fetch_add(1, std::memory_order_relaxed) & 0xfffffu;
                    while (p.dec_tag == 0);
                }
            }
            return launch_decode(p, args->dtype, s->s);  // records main_done itself, before the combine
        }
        default: set_error("internal: no kernel for id %d", id); return FHIP_ERR_UNSUPPORTED;
    }
    if (rc == FHIP_OK) FHIP_MARK_MAIN_DONE(p, s->s);
    return rc;
}

int fhip_calibration_mfma(fhip_stream *s, fhip_dtype dtype, int32_t random_operands, int32_t duty_percent, int32_t rounds,
                          void *scratch, size_t scratch_bytes) {
    if (!s || !scratch) {
        set_error("calibration: NULL stream or scratch");
        return FHIP_ERR_INVALID_ARG;
    }
    if (duty_percent < 40 || duty_percent > 100 || rounds < 1 || rounds > FHIP_CALIBRATION_MFMA_MAX_ROUNDS) {
        set_error("calibration: duty_percent %d must be in 40..100 and rounds %d in 1..%d", duty_percent, rounds,
                  FHIP_CALIBRATION_MFMA_MAX_ROUNDS);
        return FHIP_ERR_INVALID_ARG;
    }
    const int cus = s->dev->prop.multiProcessorCount;
    if (scratch_bytes < calibration_mfma_bytes(cus) || ((uintptr_t)scratch & 15) != 0) {
        set_error("calibration: scratch of %zu bytes, 16-byte aligned, needed (got %zu)", calibration_mfma_bytes(cus), scratch_bytes);
        return FHIP_ERR_WORKSPACE;
    }
    FHIP_HIP_CHECK(hipSetDevice(s->dev->ordinal));
    return launch_calibration_mfma(dtype, cus, duty_percent, rounds, random_operands ? 1 : 0, scratch, s->s);
}

int fhip_calibration_issue(fhip_stream *s, int32_t mix, int32_t rounds, void *scratch, size_t scratch_bytes) {
    if (!s || !scratch) {
        set_error("calibration: NULL stream or scratch");
        return FHIP_ERR_INVALID_ARG;
    }
    if (mix < 0 || mix >= FHIP_CALIBRATION_ISSUE_MIXES || rounds < 1 || rounds > FHIP_CALIBRATION_MFMA_MAX_ROUNDS) {
        set_error("calibration: mix %d must be in 0..%d and rounds %d in 1..%d", mix, FHIP_CALIBRATION_ISSUE_MIXES - 1, rounds,
                  FHIP_CALIBRATION_MFMA_MAX_ROUNDS);
        return FHIP_ERR_INVALID_ARG;
    }
    const int cus = s->dev->prop.multiProcessorCount;
    if (scratch_bytes < calibration_mfma_bytes(cus) || ((uintptr_t)scratch & 15) != 0) {
        set_error("calibration: scratch of %zu bytes, 16-byte aligned, needed (got %zu)", calibration_mfma_bytes(cus), scratch_bytes);
        return FHIP_ERR_WORKSPACE;
    }
    FHIP_HIP_CHECK(hipSetDevice(s->dev->ordinal));
    return launch_calibration_issue(mix, cus, rounds, scratch, s->s);
}

int fhip_calibration_xcd_map(fhip_stream *s, uint32_t workgroups, void *out, size_t out_bytes) {
    if (!s || !out || workgroups == 0 || workgroups > (1u << 20) || out_bytes < workgroups) {
        set_error("calibration: NULL stream or out, or not 1..2^20 workgroups with a byte of `out` each");
        return FHIP_ERR_INVALID_ARG;
    }
    FHIP_HIP_CHECK(hipSetDevice(s->dev->ordinal));
    return fhip::launch_xcd_probe((uint8_t *)out, (int)workgroups, s->s);
}

int fhip_calibration_read(fhip_stream *s, const void *src, size_t bytes, void *scratch, size_t scratch_bytes) {
    if (!s || !src || !scratch) {
        set_error("calibration: NULL stream, source or scratch");
        return FHIP_ERR_INVALID_ARG;
    }
    const int cus = s->dev->prop.multiProcessorCount;
    if (((uintptr_t)src & 15) != 0 || scratch_bytes < (size_t)cus * 8 * sizeof(uint32_t)) {
        set_error("calibration: the source must be 16-byte aligned and the scratch hold %zu bytes", (size_t)cus * 8 * sizeof(uint32_t));
        return FHIP_ERR_WORKSPACE;
    }
    FHIP_HIP_CHECK(hipSetDevice(s->dev->ordinal));
    return launch_calibration_read(src, bytes, cus, scratch, s->s);
}

// The same call on the library's own workspace (see `scratch` above): no hipMalloc / hipFree here or in anything
// this calls, and none needed from the caller beyond the tensors.
int fhip_flash_attention_noalloc(fhip_stream *s, const fhip_attn_args *args) {
    if (!s) {
        set_error("stream is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    size_t need = 0;
    int rc = fhip_flash_attention_workspace_bytes(args, s->dev->prop.multiProcessorCount, &need);
    if (rc) return rc;
    // What a call cannot do without: the split-KV partials of a decode step, the interval table of a mask tensor.  The
    // partials of a tiled prefill call's key split are optional: fhip_flash_attention takes the largest split that fits
    // the workspace it is given (none, if not even two shares fit).
    int32_t id;
    rc = select_kernel(args, &id, true);
    if (rc) return rc;
    if ((id == FHIP_KERNEL_PREFILL_MFMA || id == FHIP_KERNEL_PREFILL_F32) && !output_is_empty(args) && !no_keys(args))
        need = mask_scratch_bytes(args);
    if (need > STATIC_WORKSPACE_BYTES) {
        set_error("this call needs a workspace of %zu bytes; fhip_flash_attention_noalloc holds %zu (use "
                  "fhip_flash_attention with a workspace of your own)", need, STATIC_WORKSPACE_BYTES);
        return FHIP_ERR_WORKSPACE;
    }
    fhip_attn_args a = *args;
    a.workspace = s->dev->scratch_ptr;
    a.workspace_bytes = STATIC_WORKSPACE_BYTES;
    return fhip_flash_attention(s, &a);
}

// ---- masks (host, bit-exact) --------------------------------------------------------------------

static inline void put_mask(void *out, fhip_dtype dt, uint64_t idx, bool masked) {
    switch (dt) {
        case FHIP_F32: ((uint32_t *)out)[idx] = masked ? 0xFF800000u : 0u; break;
        case FHIP_F16: ((uint16_t *)out)[idx] = masked ? 0xFC00u : 0u; break;
        case FHIP_BF16: ((uint16_t *)out)[idx] = masked ? 0xFF80u : 0u; break;
    }
}

int fhip_mask_causal(fhip_dtype dtype, uint32_t n, void *out) {
    if (!dtype_ok(dtype) || (n && !out)) {
        set_error("mask_causal: bad dtype or NULL out");
        return FHIP_ERR_INVALID_ARG;
    }
    for (uint64_t i = 0; i < n; i++)
        for (uint64_t j = 0; j < n; j++) put_mask(out, dtype, i * n + j, j > i);
    return FHIP_OK;
}

int fhip_mask_sliding_window(fhip_dtype dtype, uint32_t n, uint64_t window, void *out) {
    if (!dtype_ok(dtype) || (n && !out)) {
        set_error("mask_sliding_window: bad dtype or NULL out");
        return FHIP_ERR_INVALID_ARG;
    }
    for (uint64_t i = 0; i < n; i++)
        for (uint64_t j = 0; j < n; j++) put_mask(out, dtype, i * n + j, i < j || j + window <= i);
    return FHIP_OK;
}

static uint64_t mask_offset(uint32_t seq_len, uint64_t seqlen_offset, int32_t has_window, uint64_t window) {
    if (!has_window) return seqlen_offset;
    const uint64_t room = window > seq_len ? window - seq_len : 0;  // saturating_sub
    return seqlen_offset < room ? seqlen_offset : room;
}

int fhip_mask_get_mask_shape(uint32_t seq_len, uint64_t seqlen_offset, int32_t has_window, uint64_t window,
                             uint32_t *rows, uint64_t *cols) {
    if (!rows || !cols) {
        set_error("rows/cols is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    *rows = seq_len;
    *cols = mask_offset(seq_len, seqlen_offset, has_window, window) + seq_len;
    return FHIP_OK;
}

int fhip_mask_get_mask(fhip_dtype dtype, uint32_t seq_len, uint64_t seqlen_offset, int32_t has_window,
                       uint64_t window, void *out) {
    if (!dtype_ok(dtype) || (seq_len && !out)) {
        set_error("mask_get_mask: bad dtype or NULL out");
        return FHIP_ERR_INVALID_ARG;
    }
    const uint64_t off = mask_offset(seq_len, seqlen_offset, has_window, window);
    const uint64_t cols = off + seq_len;
    for (uint64_t i = 0; i < seq_len; i++) {
        for (uint64_t j = 0; j < off; j++) put_mask(out, dtype, i * cols + j, false);
        for (uint64_t j = 0; j < seq_len; j++) {
            const bool masked = has_window ? (i < j || j + window <= i) : (j > i);
            put_mask(out, dtype, i * cols + off + j, masked);
        }
    }
    return FHIP_OK;
}

int fhip_mask_get_mask_device(fhip_stream *s, fhip_dtype dtype, uint32_t seq_len, uint64_t seqlen_offset, int32_t has_window,
                              uint64_t window, void *out_device) {
    if (!s || !dtype_ok(dtype) || (seq_len && !out_device)) {
        set_error("mask_get_mask_device: NULL stream, bad dtype or NULL out");
        return FHIP_ERR_INVALID_ARG;
    }
    const uint64_t off = mask_offset(seq_len, seqlen_offset, has_window, window);
    FHIP_HIP_CHECK(hipSetDevice(s->dev->ordinal));
    return launch_mask_build(out_device, dtype, seq_len, off + seq_len, off, has_window ? 1 : 0, window, s->s);
}

int fhip_mask_intervals_bytes(uint32_t rows, size_t *bytes) {
    if (!bytes) {
        set_error("bytes is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    *bytes = mask_intervals_bytes((int)rows);
    return FHIP_OK;
}

int fhip_mask_intervals(fhip_stream *s, const fhip_tensor2 *mask, fhip_dtype dtype, void *table, size_t table_bytes) {
    if (!s || !mask || !dtype_ok(dtype) || !table) {
        set_error("mask_intervals: NULL argument or bad dtype");
        return FHIP_ERR_INVALID_ARG;
    }
    if (mask->shape[0] > 0x7fffffffu || mask->shape[1] > 0x7fffffffu || (mask->shape[0] && mask->shape[1] && !mask->ptr)) {
        set_error("mask_intervals: mask of [%u, %u] without a device pointer, or too large", mask->shape[0], mask->shape[1]);
        return FHIP_ERR_INVALID_ARG;
    }
    if (((uintptr_t)table & 15) != 0 || table_bytes < mask_intervals_bytes((int)mask->shape[0])) {
        set_error("mask_intervals: the table must be 16-byte aligned and hold %zu bytes (got %zu)",
                  mask_intervals_bytes((int)mask->shape[0]), table_bytes);
        return FHIP_ERR_WORKSPACE;
    }
    FHIP_HIP_CHECK(hipSetDevice(s->dev->ordinal));
    int rc = launch_fill_zero_bytes(table, 16, s->s);
    if (rc) return rc;
    AttnParams p;
    memset(&p, 0, sizeof(p));
    p.mask = (const char *)mask->ptr + mask->offset * (uint64_t)elem_bytes(dtype);
    p.ms0 = mask->stride[0];
    p.ms1 = mask->stride[1];
    p.mask_kind = FHIP_MASK_QK;  // rows of the table = rows of the tensor, whichever kind it is used as
    p.Sq = (int)mask->shape[0];
    p.Skv = (int)mask->shape[1];
    p.bad_tag = MASK_TABLE_BAD;
    return launch_mask_intervals(p, dtype, (int2 *)((char *)table + 16), (int32_t *)table, s->s);
}

int fhip_mask_get_analytic(uint32_t seq_len, uint64_t seqlen_offset, int32_t has_window, uint64_t window,
                           fhip_analytic_mask *out) {
    if (!out) {
        set_error("out is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    if (has_window && window == 0) {
        // a window of 0 masks every key of every row; there is no analytic form with window>0
        set_error("sliding window of 0 masks everything; build the dense mask instead");
        return FHIP_ERR_UNSUPPORTED;
    }
    out->enabled = 1;
    out->causal = 1;
    out->q_pos_offset = (int64_t)mask_offset(seq_len, seqlen_offset, has_window, window);
    out->window = has_window ? (int64_t)window : 0;
    return FHIP_OK;
}

}  // extern "C"

// ---- growable KV cache on the device ---------------------------------------------------------------

struct fhip_tensor_cache_side {
    void *buf = nullptr;  // [B, Hkv, rows, D] contiguous; rows = allocated while growing, 2 * max_len once full
    size_t bytes = 0;     // size of buf
    // What a reset leaves behind: the sequence's buffer, kept for the next sequence's first buffers (the reference's
    // device recycles freed buffers through an allocation cache, fusor-ml/core/src/device.rs:305-354; hipMalloc and
    // hipFree cost more than a short prompt's whole attention call, and hipFree waits for the device).
    void *spare = nullptr;
    size_t spare_bytes = 0;
};

// Once the cache is full (max_sequence_len rows) it slides: the buffer holds 2 * max_len rows per (batch, head), the
// valid window starts at row `start`, new rows go behind it and the window moves; only when the buffer's end is
// reached are the kept rows copied back to row 0.  The caller sees exactly what the reference's truncating branch
// returns (the last max_len positions, in order, as one narrowed view), but an append moves O(new rows) bytes
// instead of re-concatenating the whole window every time (tensor_cache.rs:55-78).
struct fhip_kv_cache {
    fhip_device *dev;
    fhip_dtype dtype;
    uint64_t max_len;
    uint32_t B, Hkv, D;  // fixed by the first append
    uint64_t current, allocated;
    bool sliding = false;
    uint64_t start = 0;  // first valid row while sliding
    fhip_tensor_cache_side side[2];  // 0 = keys, 1 = values
};

static void kv_contig_strides(const fhip_kv_cache *c, uint64_t alloc, int64_t st[4]) {
    st[3] = 1;
    st[2] = c->D;
    st[1] = (int64_t)alloc * c->D;
    st[0] = (int64_t)c->Hkv * st[1];
}

static void kv_view(const fhip_kv_cache *c, void *buf, uint64_t alloc, uint64_t len, fhip_tensor4 *t, uint64_t first_row = 0) {
    t->ptr = buf;
    t->offset = first_row * c->D;
    t->shape[0] = c->B;
    t->shape[1] = c->Hkv;
    t->shape[2] = (uint32_t)len;
    t->shape[3] = c->D;
    kv_contig_strides(c, alloc, t->stride);
}

static uint64_t next_pow2(uint64_t x) {
    uint64_t p = 1;
    while (p < x) p <<= 1;
    return p;
}

// How the new rows of an append reach the cache: copied as they are (src_dtype == cache dtype, no
// tables), or converted on the way, the keys rotated by the rotary embedding first.
struct NewRows {
    fhip_dtype src_dtype;
    const fhip_rope_tables *rope;  // nullptr: plain copy
    const fhip_rms_norm *k_norm;   // with rope: the keys are normalised first (nullptr: not)
    fhip::RowJobs *batch;          // not nullptr: the rotated / converted rows are queued here instead of launched
};

// rows [first, first + count) of the new block `src` -> dst (cache dtype, strides dst_st); side 0 = keys
static int write_new_rows(const fhip_kv_cache *c, hipStream_t st, int side, const fhip_tensor4 *src, uint64_t first,
                          uint32_t count, void *dst, const int64_t dst_st[4], const NewRows &nr) {
    const uint32_t shp[4] = {c->B, c->Hkv, count, c->D};
    const int seb = fhip::elem_bytes(nr.src_dtype);
    const char *sp = (const char *)src->ptr + (src->offset + first * src->stride[2]) * (uint64_t)seb;
    if (!nr.rope) return launch_copy_rows(sp, src->stride, dst, dst_st, shp, seb, st);
    const int mode = side == 0 ? (nr.rope->interleaved ? 1 : 0) : 2;
    fhip::RowNorm norm;
    if (side == 0 && nr.k_norm) norm = {nr.k_norm->weight, nr.k_norm->bias, nr.k_norm->dtype, nr.k_norm->eps};
    if (nr.batch && nr.batch->n < 3) {
        fhip::fill_row_job(&nr.batch->job[nr.batch->n++], sp, src->stride, nr.src_dtype, dst, dst_st, c->dtype, shp,
                           nr.rope->cos, nr.rope->sin, (int64_t)(nr.rope->start_pos + first), mode,
                           side == 0 && nr.k_norm ? &norm : nullptr);
        return FHIP_OK;
    }
    return launch_rope_rows(sp, src->stride, nr.src_dtype, dst, dst_st, c->dtype, shp, nr.rope->cos, nr.rope->sin,
                            (int64_t)(nr.rope->start_pos + first), mode, side == 0 && nr.k_norm ? &norm : nullptr, st);
}

extern "C" {

int fhip_kv_cache_create(fhip_device *dev, fhip_dtype dtype, uint64_t max_sequence_len, fhip_kv_cache **out) {
    if (!dev || !out || !fhip::dtype_ok(dtype)) {
        set_error("kv_cache_create: NULL argument or bad dtype");
        return FHIP_ERR_INVALID_ARG;
    }
    if (max_sequence_len == 0 || max_sequence_len > 0x7fffffffull) {
        set_error("kv_cache_create: max_sequence_len must be in 1..2^31-1");
        return FHIP_ERR_INVALID_ARG;
    }
    fhip_kv_cache *c = new (std::nothrow) fhip_kv_cache();
    if (!c) {
        set_error("out of host memory");
        return FHIP_ERR_HIP;
    }
    c->dev = dev;
    c->dtype = dtype;
    c->max_len = max_sequence_len;
    c->B = c->Hkv = c->D = 0;
    c->current = c->allocated = 0;
    *out = c;
    return FHIP_OK;
}

// keep_memory: the larger of the current buffer and the spare stays with the cache as its spare
static int kv_release(fhip_kv_cache *c, bool keep_memory) {
    int rc = FHIP_OK;
    if (hipSetDevice(c->dev->ordinal) != hipSuccess) rc = FHIP_ERR_HIP;
    for (int s = 0; s < 2; s++) {
        fhip_tensor_cache_side &S = c->side[s];
        if (keep_memory && S.buf && S.bytes > S.spare_bytes) {
            void *smaller = S.spare;
            S.spare = S.buf, S.spare_bytes = S.bytes;
            S.buf = smaller;
        }
        if (S.buf && hipFree(S.buf) != hipSuccess) rc = FHIP_ERR_HIP;
        S.buf = nullptr, S.bytes = 0;
        if (!keep_memory) {
            if (S.spare && hipFree(S.spare) != hipSuccess) rc = FHIP_ERR_HIP;
            S.spare = nullptr, S.spare_bytes = 0;
        }
    }
    c->current = c->allocated = 0;
    c->sliding = false;
    c->start = 0;
    c->B = c->Hkv = c->D = 0;
    if (rc) set_error("kv_cache: hipFree failed");
    return rc;
}

int fhip_kv_cache_destroy(fhip_kv_cache *c) {
    if (!c) return FHIP_OK;
    int rc = kv_release(c, false);
    delete c;
    return rc;
}

// TensorCache::reset (tensor_cache.rs:39-43): drops the data, keeps the limits (and the memory, for the next sequence).
int fhip_kv_cache_reset(fhip_kv_cache *c) {
    if (!c) {
        set_error("cache is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    return kv_release(c, true);
}

int fhip_kv_cache_current_seq_len(const fhip_kv_cache *c, uint64_t *len) {
    if (!c || !len) {
        set_error("cache/len is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    *len = c->current;
    return FHIP_OK;
}

int fhip_kv_cache_allocated_seq_len(const fhip_kv_cache *c, uint64_t *len) {
    if (!c || !len) {
        set_error("cache/len is NULL");
        return FHIP_ERR_INVALID_ARG;
    }
    *len = c->allocated;
    return FHIP_OK;
}

static int kv_append_core(fhip_kv_cache *c, fhip_stream *s, const fhip_tensor4 *k_new, const fhip_tensor4 *v_new,
                          fhip_tensor4 *k_all, fhip_tensor4 *v_all, const NewRows &nr) {
    if (!c || !s || !k_new || !v_new || !k_all || !v_all) {
        set_error("kv_cache_append: NULL argument");
        return FHIP_ERR_INVALID_ARG;
    }
    if (!k_new->ptr || !v_new->ptr) {
        set_error("kv_cache_append: new keys/values need device pointers");
        return FHIP_ERR_INVALID_ARG;
    }
    for (int i = 0; i < 4; i++) {
        if (k_new->shape[i] != v_new->shape[i]) {
            set_error("kv_cache_append: key shape [%u, %u, %u, %u] != value shape [%u, %u, %u, %u]", k_new->shape[0],
                      k_new->shape[1], k_new->shape[2], k_new->shape[3], v_new->shape[0], v_new->shape[1],
                      v_new->shape[2], v_new->shape[3]);
            return FHIP_ERR_INVALID_ARG;
        }
        if (k_new->shape[i] == 0) {
            set_error("kv_cache_append: empty tensor");
            return FHIP_ERR_INVALID_ARG;
        }
    }
    const bool first = c->side[0].buf == nullptr;
    if (!first && (k_new->shape[0] != c->B || k_new->shape[1] != c->Hkv || k_new->shape[3] != c->D)) {
        set_error("kv_cache_append: [%u, %u, _, %u] does not match the cached [%u, %u, _, %u]", k_new->shape[0],
                  k_new->shape[1], k_new->shape[3], c->B, c->Hkv, c->D);
        return FHIP_ERR_INVALID_ARG;
    }
    FHIP_HIP_CHECK(hipSetDevice(c->dev->ordinal));
    const int eb = fhip::elem_bytes(c->dtype);
    const uint64_t n = k_new->shape[2];
    const uint64_t required = c->current + n;
    if (first) {
        c->B = k_new->shape[0];
        c->Hkv = k_new->shape[1];
        c->D = k_new->shape[3];
    }
    const size_t row_elems = (size_t)c->B * c->Hkv * c->D;
    const fhip_tensor4 *news[2] = {k_new, v_new};
    fhip_tensor4 *alls[2] = {k_all, v_all};

    // Branches that move the cache into new buffers allocate both sides' buffers before anything is queued and
    // install them only after every launch into them was accepted: a failure on the way frees them and leaves the
    // cache (buffers, lengths, strides) exactly as it was.
    void *nb[2] = {nullptr, nullptr};
    size_t nb_bytes[2] = {0, 0};
    auto drop_new = [&]() {
        for (int sd = 0; sd < 2; sd++)
            if (nb[sd]) (void)hipFree(nb[sd]);
    };
    auto alloc_new = [&](size_t bytes) -> int {
        for (int sd = 0; sd < 2; sd++) {
            fhip_tensor_cache_side &S = c->side[sd];
            if (S.spare && S.spare_bytes >= bytes) {  // what the last reset left (work queued on this stream before the
                nb[sd] = S.spare;                      // reset is done with it before anything queued now writes to it)
                nb_bytes[sd] = S.spare_bytes;
                S.spare = nullptr, S.spare_bytes = 0;
                continue;
            }
            const hipError_t e = hipMalloc(&nb[sd], bytes);
            if (e != hipSuccess) {
                nb[sd] = nullptr;
                drop_new();
                return fhip::hip_fail(e, "hipMalloc (KV cache buffers)");
            }
            nb_bytes[sd] = bytes;
        }
        return FHIP_OK;
    };
    auto install_new = [&]() {
        for (int sd = 0; sd < 2; sd++) {
            if (c->side[sd].buf) (void)hipFree(c->side[sd].buf);  // waits for the copies out of it
            c->side[sd].buf = nb[sd];
            c->side[sd].bytes = nb_bytes[sd];
        }
    };

    if (required > c->max_len) {
        // keep the last max_len positions of old[new_start..] ++ new (tensor_cache.rs:55-78)
        const uint64_t mx = c->max_len, cap = 2 * mx;
        const uint64_t new_start = required - mx;  // rows dropped from the front of old ++ new
        const uint64_t keep_old = c->current > new_start ? c->current - new_start : 0;  // rows kept from the cache
        const uint64_t take_new = mx - keep_old;                                          // last rows of the new block
        const bool behind = c->sliding && c->start + c->current + n <= cap;  // room behind the window: nothing moves
        int64_t cap_st[4];
        kv_contig_strides(c, cap, cap_st);
        uint64_t start_after = 0;
        if (!c->sliding) {
            // the cache has just filled up: move what is kept into buffers with room to slide
            int rc = alloc_new(row_elems * cap * eb);
            if (rc) return rc;
            for (int sd = 0; sd < 2 && !rc; sd++) {
                if (keep_old) {
                    int64_t src_st[4];
                    kv_contig_strides(c, c->allocated, src_st);
                    const uint32_t shp[4] = {c->B, c->Hkv, (uint32_t)keep_old, c->D};
                    rc = launch_copy_rows((const char *)c->side[sd].buf + new_start * c->D * eb, src_st, nb[sd], cap_st, shp,
                                          eb, s->s);
                }
                if (!rc)
                    rc = write_new_rows(c, s->s, sd, news[sd], n - take_new, (uint32_t)take_new,
                                        (char *)nb[sd] + keep_old * c->D * eb, cap_st, nr);
            }
            if (rc) {
                (void)hipStreamSynchronize(s->s);  // nothing queued may still write into the buffers being dropped
                drop_new();
                if (first) c->B = c->Hkv = c->D = 0;  // still empty
                return rc;
            }
            install_new();
        } else {
            for (int sd = 0; sd < 2; sd++) {
                fhip_tensor_cache_side &S = c->side[sd];
                if (behind) {
                    // keep_old > 0 here, so every new row is kept
                    int rc = write_new_rows(c, s->s, sd, news[sd], 0, (uint32_t)n,
                                            (char *)S.buf + (c->start + c->current) * c->D * eb, cap_st, nr);
                    if (rc) return rc;
                    start_after = c->start + new_start;
                } else {
                    // the end of the buffer: the kept rows go back to row 0 (they lie beyond row max_len - n, so source
                    // and destination do not overlap), the new ones behind them
                    if (keep_old) {
                        const uint32_t shp[4] = {c->B, c->Hkv, (uint32_t)keep_old, c->D};
                        int rc = launch_copy_rows((const char *)S.buf + (c->start + new_start) * c->D * eb, cap_st, S.buf,
                                                  cap_st, shp, eb, s->s);
                        if (rc) return rc;
                    }
                    int rc = write_new_rows(c, s->s, sd, news[sd], n - take_new, (uint32_t)take_new,
                                            (char *)S.buf + keep_old * c->D * eb, cap_st, nr);
                    if (rc) return rc;
                    start_after = 0;
                }
            }
        }
        for (int sd = 0; sd < 2; sd++) kv_view(c, c->side[sd].buf, cap, mx, alls[sd], start_after);
        c->sliding = true;
        c->start = start_after;
        c->current = mx;
        c->allocated = mx;
        return FHIP_OK;
    }

    if (first) {
        // first append stores the tensor as it is (tensor_cache.rs:111-116)
        int rc = alloc_new(row_elems * n * eb);
        int64_t dst_st[4];
        kv_contig_strides(c, n, dst_st);
        for (int sd = 0; sd < 2 && !rc; sd++) rc = write_new_rows(c, s->s, sd, news[sd], 0, (uint32_t)n, nb[sd], dst_st, nr);
        if (rc) {
            (void)hipStreamSynchronize(s->s);
            drop_new();
            c->B = c->Hkv = c->D = 0;  // still empty
            return rc;
        }
        install_new();
        for (int sd = 0; sd < 2; sd++) kv_view(c, c->side[sd].buf, n, n, alls[sd]);
        c->current = n;
        c->allocated = n;
        return FHIP_OK;
    }

    uint64_t alloc = c->allocated;
    if (required > c->allocated) alloc = next_pow2(required);  // tensor_cache.rs:80-96
    int64_t dst_st[4];
    kv_contig_strides(c, alloc, dst_st);
    if (alloc != c->allocated) {
        int rc = alloc_new(row_elems * alloc * eb);
        if (rc) return rc;
        int64_t src_st[4];
        kv_contig_strides(c, c->allocated, src_st);
        for (int sd = 0; sd < 2 && !rc; sd++) {
            const uint32_t shp_old[4] = {c->B, c->Hkv, (uint32_t)c->current, c->D};
            rc = launch_copy_rows(c->side[sd].buf, src_st, nb[sd], dst_st, shp_old, eb, s->s);
            if (!rc && alloc > required) {  // the reference concatenates zeros behind the data
                const uint32_t shp_z[4] = {c->B, c->Hkv, (uint32_t)(alloc - required), c->D};
                rc = launch_fill_zero_rows((char *)nb[sd] + required * c->D * eb, dst_st, shp_z, eb, s->s);
            }
            if (!rc)
                rc = write_new_rows(c, s->s, sd, news[sd], 0, (uint32_t)n, (char *)nb[sd] + c->current * c->D * eb, dst_st, nr);
        }
        if (rc) {
            (void)hipStreamSynchronize(s->s);
            drop_new();
            return rc;
        }
        install_new();
    } else {
        for (int sd = 0; sd < 2; sd++) {
            int rc = write_new_rows(c, s->s, sd, news[sd], 0, (uint32_t)n, (char *)c->side[sd].buf + c->current * c->D * eb,
                                    dst_st, nr);
            if (rc) return rc;
        }
    }
    for (int sd = 0; sd < 2; sd++) kv_view(c, c->side[sd].buf, alloc, required, alls[sd]);
    c->current = required;
    c->allocated = alloc;
    return FHIP_OK;
}

int fhip_kv_cache_append(fhip_kv_cache *c, fhip_stream *s, const fhip_tensor4 *k_new, const fhip_tensor4 *v_new,
                         fhip_tensor4 *k_all, fhip_tensor4 *v_all) {
    NewRows nr;
    nr.src_dtype = c ? c->dtype : FHIP_F32;
    nr.rope = nullptr;
    nr.k_norm = nullptr;
    nr.batch = nullptr;
    return kv_append_core(c, s, k_new, v_new, k_all, v_all, nr);
}

static int check_rope(const fhip_rope_tables *r, uint32_t head_dim, uint64_t rows) {
    if (!r || !r->cos || !r->sin) {
        set_error("rope: NULL tables");
        return FHIP_ERR_INVALID_ARG;
    }
    if (head_dim == 0 || head_dim % 2 != 0) {
        set_error("rope: head_dim %u must be even", head_dim);
        return FHIP_ERR_INVALID_ARG;
    }
    if (r->start_pos + rows > r->table_rows) {
        set_error("rope: positions %llu..%llu exceed the %llu rows of the tables", (unsigned long long)r->start_pos,
                  (unsigned long long)(r->start_pos + rows), (unsigned long long)r->table_rows);
        return FHIP_ERR_INVALID_ARG;
    }
    return FHIP_OK;
}

static int check_norm(const fhip_rms_norm *n) {
    if (!n || !n->weight || !fhip::dtype_ok(n->dtype)) {
        set_error("rms norm: NULL weight or bad dtype");
        return FHIP_ERR_INVALID_ARG;
    }
    return FHIP_OK;
}

static int rope_core(fhip_stream *s, const fhip_rms_norm *norm, const fhip_rope_tables *rope, const fhip_tensor4 *x,
                     fhip_dtype x_dtype, const fhip_tensor4 *out, fhip_dtype out_dtype) {
    if (!s || !x || !out || !x->ptr || !out->ptr || !fhip::dtype_ok(x_dtype) || !fhip::dtype_ok(out_dtype)) {
        set_error("rope: NULL argument or bad dtype");
        return FHIP_ERR_INVALID_ARG;
    }
    for (int i = 0; i < 4; i++)
        if (x->shape[i] != out->shape[i]) {
            set_error("rope: output shape differs from the input shape");
            return FHIP_ERR_INVALID_ARG;
        }
    int rc = FHIP_OK;
    if (rope) rc = check_rope(rope, x->shape[3], x->shape[2]);
    else if (x->shape[3] == 0 || x->shape[3] % 2 != 0) {
        set_error("rms norm: head_dim %u must be even", x->shape[3]);
        rc = FHIP_ERR_INVALID_ARG;
    }
    if (rc) return rc;
    fhip::RowNorm rn;
    if (norm) {
        rc = check_norm(norm);
        if (rc) return rc;
        rn = {norm->weight, norm->bias, norm->dtype, norm->eps};
    }
    FHIP_HIP_CHECK(hipSetDevice(s->dev->ordinal));
    const char *sp = (const char *)x->ptr + x->offset * (uint64_t)fhip::elem_bytes(x_dtype);
    char *dp = (char *)out->ptr + out->offset * (uint64_t)fhip::elem_bytes(out_dtype);
    return launch_rope_rows(sp, x->stride, x_dtype, dp, out->stride, out_dtype, x->shape, rope ? rope->cos : nullptr,
                            rope ? rope->sin : nullptr, rope ? (int64_t)rope->start_pos : 0,
                            rope ? (rope->interleaved ? 1 : 0) : 2, norm ? &rn : nullptr, s->s);
}

int fhip_rope(fhip_stream *s, const fhip_rope_tables *rope, const fhip_tensor4 *x, fhip_dtype x_dtype, const fhip_tensor4 *out,
              fhip_dtype out_dtype) {
    if (!rope) {
        set_error("rope: NULL tables");
        return FHIP_ERR_INVALID_ARG;
    }
    return rope_core(s, nullptr, rope, x, x_dtype, out, out_dtype);
}

int fhip_norm_rope(fhip_stream *s, const fhip_rms_norm *norm, const fhip_rope_tables *rope, const fhip_tensor4 *x,
                   fhip_dtype x_dtype, const fhip_tensor4 *out, fhip_dtype out_dtype) {
    int rc = check_norm(norm);
    if (rc) return rc;
    return rope_core(s, norm, rope, x, x_dtype, out, out_dtype);
}

static int rope_append_core(fhip_kv_cache *c, fhip_stream *s, const fhip_rms_norm *k_norm, const fhip_rope_tables *rope,
                            const fhip_tensor4 *k_new, const fhip_tensor4 *v_new, fhip_dtype in_dtype, fhip_tensor4 *k_all,
                            fhip_tensor4 *v_all, fhip::RowJobs *batch = nullptr) {
    if (!k_new || !fhip::dtype_ok(in_dtype)) {
        set_error("kv_cache_rope_append: NULL argument or bad dtype");
        return FHIP_ERR_INVALID_ARG;
    }
    int rc = check_rope(rope, k_new->shape[3], k_new->shape[2]);
    if (rc) return rc;
    NewRows nr;
    nr.src_dtype = in_dtype;
    nr.rope = rope;
    nr.k_norm = k_norm;
    nr.batch = batch;
    return kv_append_core(c, s, k_new, v_new, k_all, v_all, nr);
}

int fhip_kv_cache_rope_append(fhip_kv_cache *c, fhip_stream *s, const fhip_rope_tables *rope, const fhip_tensor4 *k_new,
                              const fhip_tensor4 *v_new, fhip_dtype in_dtype, fhip_tensor4 *k_all, fhip_tensor4 *v_all) {
    return rope_append_core(c, s, nullptr, rope, k_new, v_new, in_dtype, k_all, v_all);
}

int fhip_kv_cache_qkv_rope_append(fhip_kv_cache *c, fhip_stream *s, const fhip_rms_norm *q_norm, const fhip_rms_norm *k_norm,
                                  const fhip_rope_tables *rope, const fhip_tensor4 *q, fhip_dtype q_dtype,
                                  const fhip_tensor4 *q_out, fhip_dtype q_out_dtype, const fhip_tensor4 *k_new,
                                  const fhip_tensor4 *v_new, fhip_dtype in_dtype, fhip_tensor4 *k_all, fhip_tensor4 *v_all) {
    if (!s || !q || !q_out || !q->ptr || !q_out->ptr || !fhip::dtype_ok(q_dtype) || !fhip::dtype_ok(q_out_dtype)) {
        set_error("kv_cache_qkv_rope_append: NULL argument or bad dtype");
        return FHIP_ERR_INVALID_ARG;
    }
    for (int i = 0; i < 4; i++)
        if (q->shape[i] != q_out->shape[i]) {
            set_error("kv_cache_qkv_rope_append: q_out shape differs from q's");
            return FHIP_ERR_INVALID_ARG;
        }
    int rc = check_rope(rope, q->shape[3], q->shape[2]);
    if (rc) return rc;
    if (q_norm && (rc = check_norm(q_norm))) return rc;
    if (k_norm && (rc = check_norm(k_norm))) return rc;
    fhip::RowJobs jobs;
    jobs.n = 0;
    fhip::RowNorm qn;
    if (q_norm) qn = {q_norm->weight, q_norm->bias, q_norm->dtype, q_norm->eps};
    const char *qp = (const char *)q->ptr + q->offset * (uint64_t)fhip::elem_bytes(q_dtype);
    char *qo = (char *)q_out->ptr + q_out->offset * (uint64_t)fhip::elem_bytes(q_out_dtype);
    fhip::fill_row_job(&jobs.job[jobs.n++], qp, q->stride, q_dtype, qo, q_out->stride, q_out_dtype, q->shape, rope->cos,
                       rope->sin, (int64_t)rope->start_pos, rope->interleaved ? 1 : 0, q_norm ? &qn : nullptr);
    // the cache bookkeeping (growth, truncation, their copies) runs as usual; the new rows join q's launch
    rc = rope_append_core(c, s, k_norm, rope, k_new, v_new, in_dtype, k_all, v_all, &jobs);
    if (rc) return rc;
    return launch_row_jobs(jobs, s->s);
}

int fhip_kv_cache_norm_rope_append(fhip_kv_cache *c, fhip_stream *s, const fhip_rms_norm *k_norm,
                                   const fhip_rope_tables *rope, const fhip_tensor4 *k_new, const fhip_tensor4 *v_new,
                                   fhip_dtype in_dtype, fhip_tensor4 *k_all, fhip_tensor4 *v_all) {
    int rc = check_norm(k_norm);
    if (rc) return rc;
    return rope_append_core(c, s, k_norm, rope, k_new, v_new, in_dtype, k_all, v_all);
}

}  // extern "C"
