/*
 * TEST INFRASTRUCTURE ONLY -- never linked into, imported by or called from the shipped library.
 *
 * CPU restatement, in plain C, of fusor-ml's CPU attention composite
 * (reference: fusor-ml/fusor/src/composite/flash_attention.rs:77-200).  It is the checker the
 * HIP kernels are compared with, and the "port" CPU baseline the benchmark times.
 *
 * Every value is IEEE-754 binary32 and every step is one rounding, in the order the reference
 * performs them:
 *   1. GQA head mapping  kv_head = head / (H / Hkv)          flash_attention.rs:101-138
 *   2. K^T materialised, scores = Q @ K^T                    flash_attention.rs:141-142
 *      (row-major GEMM, f32 FMA accumulation along the contraction index in increasing order;
 *       fusor-ml/cpu/src/matmul.rs:51-73 hands this to the `gemm` crate 0.18.2, whose
 *       micro-kernel order is not part of the reference tree: bit-level GEMM parity is UNPINNED,
 *       value-level parity is pinned by the float64 twin and the closed forms in tests/)
 *   3. scores * scale as a separate multiply                 flash_attention.rs:145
 *   4. scores + mask (additive, QKMask [Sq,Skv] or BatchKeyMask [B,Skv])   :148-180
 *   5. m = left-to-right fold of max starting at -inf        flash_attention.rs:184-189,
 *                                                            fusor-ml/cpu/src/reduce.rs:178-183,700-764
 *   6. e = expf(s - m)                                       :189-191, fusor-ml/cpu/src/elementwise.rs:157
 *   7. l = left-to-right fold of + starting at 0             :192-195
 *   8. p = e / l  (true division)                            :196
 *   9. out = P @ V  (same GEMM)                              :199
 *
 * Parity status of each function is stated where it is defined.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_MASK_NONE 0
#define ORACLE_MASK_QK 1
#define ORACLE_MASK_BATCH_KEY 2

/* f32::max of the Rust standard library: returns the non-NaN operand when exactly one is NaN
 * (fusor-ml/cpu/src/reduce.rs:182 uses it through MaxOp). */
static inline float rust_f32_max(float a, float b) {
    if (a != a) return b;
    if (b != b) return a;
    return a > b ? a : b;
}

/* C[m, 0..N) = sum_k A[m,k] * Bt[k, 0..N)   with one fused multiply-add per term, k increasing.
 * Outer-product form so the compiler vectorises across N without reassociating the k-sum. */
static void gemm_row_f32(const float *a_row, int K, const float *b, long ldb, int N, float *c_row) {
    for (int n = 0; n < N; n++) c_row[n] = 0.0f;
    for (int k = 0; k < K; k++) {
        const float a = a_row[k];
        const float *brow = b + (long)k * ldb;
        for (int n = 0; n < N; n++) c_row[n] = fmaf(a, brow[n], c_row[n]);
    }
}

/*
 * oracle_flash_attention_f32 -- parity: PINNED at value level (float64 twin to 1e-6 rel-L2,
 * closed forms: causal row 0 == V[0], equal scores => mean of V, single key => V row, mask-row
 * shift invariance, -inf BatchKeyMask padding == unpadded call; the reference's own 2x2 causal
 * test flash_attention.rs:241-276).  Bit-level GEMM order UNPINNED (see header).
 *
 * q [B,H,Sq,D], k,v [B,Hkv,Skv,D], contiguous row-major f32.  mask: NULL or contiguous f32.
 * rows: NULL -> every query row, out is [B,H,Sq,D]; else `nrows` query-row indices (each row is
 * independent of the others in the reference algorithm), out is [B,H,nrows,D].
 * Returns 0, or -1 on the argument errors the reference asserts on (H % Hkv != 0).
 */
int oracle_flash_attention_f32(const float *q, const float *k, const float *v, const float *mask,
                               int mask_kind, int B, int H, int Hkv, int Sq, int Skv, int D,
                               float scale, const int32_t *rows, int nrows, float *out,
                               int nthreads) {
    if (Hkv <= 0 || H % Hkv != 0) return -1; /* flash_attention.rs:94-99 */
    const int G = H / Hkv;
    const int R = rows ? nrows : Sq;
    int failed = 0;
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#endif
    (void)nthreads;
    /* one (batch, kv head) at a time so K^T is built once for its G query heads */
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int b = 0; b < B; b++) {
        for (int g = 0; g < Hkv; g++) {
            const float *kg = k + ((long)b * Hkv + g) * (long)Skv * D;
            const float *vg = v + ((long)b * Hkv + g) * (long)Skv * D;
            float *kt = (float *)malloc(sizeof(float) * (size_t)D * (size_t)(Skv > 0 ? Skv : 1));
            float *s = (float *)malloc(sizeof(float) * (size_t)(Skv > 0 ? Skv : 1));
            if (!kt || !s) {
                failed = 1;
                free(kt);
                free(s);
                continue;
            }
            for (int j = 0; j < Skv; j++) /* k_t = K.transpose(2,3), materialised (:141) */
                for (int d = 0; d < D; d++) kt[(long)d * Skv + j] = kg[(long)j * D + d];
            for (int hh = 0; hh < G; hh++) {
                const int h = g * G + hh; /* kv head of h is h / G == g */
                for (int r = 0; r < R; r++) {
                    const int i = rows ? rows[r] : r;
                    const float *qrow = q + (((long)b * H + h) * Sq + i) * D;
                    gemm_row_f32(qrow, D, kt, Skv, Skv, s);
                    for (int j = 0; j < Skv; j++) s[j] = s[j] * scale;
                    if (mask_kind == ORACLE_MASK_QK) {
                        const float *mrow = mask + (long)i * Skv;
                        for (int j = 0; j < Skv; j++) s[j] = s[j] + mrow[j];
                    } else if (mask_kind == ORACLE_MASK_BATCH_KEY) {
                        const float *mrow = mask + (long)b * Skv;
                        for (int j = 0; j < Skv; j++) s[j] = s[j] + mrow[j];
                    }
                    float m = -INFINITY;
                    for (int j = 0; j < Skv; j++) m = rust_f32_max(m, s[j]);
                    for (int j = 0; j < Skv; j++) s[j] = expf(s[j] - m);
                    float l = 0.0f;
                    for (int j = 0; j < Skv; j++) l = l + s[j];
                    for (int j = 0; j < Skv; j++) s[j] = s[j] / l;
                    float *orow = out + (((long)b * H + h) * R + r) * D;
                    gemm_row_f32(s, Skv, vg, D, D, orow);
                }
            }
            free(kt);
            free(s);
        }
    }
    return failed ? -2 : 0;
}

/*
 * The same nine steps written as naively as possible (scalar triple loops, separate score
 * matrix).  Used only to cross-check oracle_flash_attention_f32 on small inputs: the two share
 * no loop structure, so an indexing mistake in one does not hide in the other.
 * parity: PINNED with the same checks as above.
 */
int oracle_flash_attention_naive_f32(const float *q, const float *k, const float *v,
                                     const float *mask, int mask_kind, int B, int H, int Hkv,
                                     int Sq, int Skv, int D, float scale, float *out) {
    if (Hkv <= 0 || H % Hkv != 0) return -1;
    const int G = H / Hkv;
    float *s = (float *)malloc(sizeof(float) * (size_t)(Sq > 0 ? Sq : 1) * (size_t)(Skv > 0 ? Skv : 1));
    if (!s) return -2;
    for (int b = 0; b < B; b++)
        for (int h = 0; h < H; h++) {
            const int g = h / G;
            for (int i = 0; i < Sq; i++)
                for (int j = 0; j < Skv; j++) {
                    float acc = 0.0f;
                    for (int d = 0; d < D; d++)
                        acc = fmaf(q[(((long)b * H + h) * Sq + i) * D + d],
                                   k[(((long)b * Hkv + g) * Skv + j) * D + d], acc);
                    acc = acc * scale;
                    if (mask_kind == ORACLE_MASK_QK) acc = acc + mask[(long)i * Skv + j];
                    if (mask_kind == ORACLE_MASK_BATCH_KEY) acc = acc + mask[(long)b * Skv + j];
                    s[(long)i * Skv + j] = acc;
                }
            for (int i = 0; i < Sq; i++) {
                float *row = s + (long)i * Skv;
                float m = -INFINITY;
                for (int j = 0; j < Skv; j++) m = rust_f32_max(m, row[j]);
                float l = 0.0f;
                for (int j = 0; j < Skv; j++) {
                    row[j] = expf(row[j] - m);
                    l = l + row[j];
                }
                for (int j = 0; j < Skv; j++) row[j] = row[j] / l;
                for (int d = 0; d < D; d++) {
                    float acc = 0.0f;
                    for (int j = 0; j < Skv; j++)
                        acc = fmaf(row[j], v[(((long)b * Hkv + g) * Skv + j) * D + d], acc);
                    out[(((long)b * H + h) * Sq + i) * D + d] = acc;
                }
            }
        }
    free(s);
    return 0;
}

/* ---- masks: bit-exact restatements ---------------------------------------------------------
 * parity: PINNED by the reference's own vectors (attention_mask.rs:99-110 3x3 causal,
 * mask_cache.rs:139-175 shape [2,5] and the (4,0,W=2) entries,
 * interfaces/kalosm-common/src/mask.rs:69-98 golden 4x4 causal and sliding matrices). */

/* AttentionMask::causal, fusor-ml/fusor/src/cache/attention_mask.rs:26-34 */
void oracle_mask_causal_f32(int n, float *out) {
    for (int i = 0; i < n; i++)
        for (int j = 0; j < n; j++) out[(long)i * n + j] = (j > i) ? -INFINITY : 0.0f;
}

/* MaskCache::create_sliding_window_mask, fusor-ml/fusor/src/cache/mask_cache.rs:88-103 */
void oracle_mask_sliding_f32(int n, long window, float *out) {
    for (long i = 0; i < n; i++)
        for (long j = 0; j < n; j++)
            out[i * n + j] = (i < j || j + window <= i) ? -INFINITY : 0.0f;
}

/* MaskCache::get_mask offset rule, mask_cache.rs:43-49: with a window the left padding is
 * min(seqlen_offset, window.saturating_sub(seq_len)). */
long oracle_get_mask_offset(long seq_len, long seqlen_offset, int has_window, long window) {
    if (!has_window) return seqlen_offset;
    long room = window > seq_len ? window - seq_len : 0;
    return seqlen_offset < room ? seqlen_offset : room;
}

/* MaskCache::get_mask, mask_cache.rs:36-86.  out is [seq_len, offset' + seq_len]. */
void oracle_get_mask_f32(int seq_len, long seqlen_offset, int has_window, long window, float *out) {
    long off = oracle_get_mask_offset(seq_len, seqlen_offset, has_window, window);
    long cols = off + seq_len;
    for (long i = 0; i < seq_len; i++) {
        for (long j = 0; j < off; j++) out[i * cols + j] = 0.0f; /* Tensor::zeros (:79) */
        for (long j = 0; j < seq_len; j++) {
            int masked = has_window ? (i < j || j + window <= i) : (j > i);
            out[i * cols + off + j] = masked ? -INFINITY : 0.0f;
        }
    }
}
