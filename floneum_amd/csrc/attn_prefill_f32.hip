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
// Short prompts leave most of the chip idle with 128 rows per workgroup, and the f32 matrix rate makes
// the longest wavefront's tile sequence the critical path.  The kernel therefore also comes in key-split
// forms (template parameter S = 2, 4): the four wavefronts form S groups that own the SAME 128 / S query
// rows, group g walks the key tiles t with t % S == g through its own LDS buffers, and the groups'
// (m, l, O) states are merged through LDS at the end.  S times the workgroups, 1 / S of the tiles each.
// With S = 4 a group is one wavefront; above head_dim 64 it cannot hold a K and a V tile in staging
// registers at once, so the two take turns in one register set and one LDS buffer, with no workgroup
// barrier inside the loop.
//
// Reference semantics: fusor-ml/fusor/src/composite/flash_attention.rs:141-199; this is the data
// type kalosm-llama always calls with (models/kalosm-llama/src/raw/attention_layer.rs:400-448).
#include "attn_bounds.h"
#include "common.h"
#include "device_utils.h"

namespace fhip {

constexpr int PF32_WAVES = 4;
constexpr int PF32_BN = 32;
constexpr float PF32_LOG2E = 1.4426950408889634f;

// four consecutive elements of a row as f32 (16-bit storage types are widened exactly)
__device__ __forceinline__ float4_t load4(const float *p) { return *(const float4_t *)p; }
__device__ __forceinline__ float4_t load4(const half_t *p) {
    const half4_t h = *(const half4_t *)p;
    return float4_t{(float)h[0], (float)h[1], (float)h[2], (float)h[3]};
}
__device__ __forceinline__ float4_t load4(const bf16_t *p) {
    const uint2_t u = *(const uint2_t *)p;
    return float4_t{__uint_as_float(u[0] << 16), __uint_as_float(u[0] & 0xffff0000u), __uint_as_float(u[1] << 16),
                    __uint_as_float(u[1] & 0xffff0000u)};
}
// one output element: the tensors' type, or f32 when the call asks for an f32 result of 16-bit inputs
template <typename T>
__device__ __forceinline__ void store_out(const AttnParams &p, int64_t idx, float v) {
    if (sizeof(T) == 4 || p.out_f32) ((float *)p.out)[idx] = v;
    else ((T *)p.out)[idx] = from_float<T>(v);
}

// odd rounds of `cus` workgroups are numbered backwards (see AttnParams::snake_cus)
__device__ __forceinline__ int snake_order(int id, int total, int cus) {
    if (cus <= 0) return id;
    const int r = id / cus, j = id % cus;
    if ((r & 1) == 0) return id;
    const int len = min(cus, total - r * cus);
    return r * cus + (len - 1 - j);
}

#define LDS32_PTR(type, byte_off) ((__attribute__((address_space(3))) type *)(lds_base + (byte_off)))

__device__ __forceinline__ float half_swap_max32(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum32(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// How a mask tensor is applied (MODE):
//   PF32_INTERVALS  by interval: analytic description, key counts, or the interval form a scan launch left in p.iv
//   PF32_BIAS       the tensor is added as it is, element by element (p.mask, no interval form): finite biases,
//                   several visible runs per row, NaN or +inf entries.  Score = (q.k * scale) + mask as in the
//                   reference (fusor flash_attention.rs:145,177), every key tile is visited.
//   PF32_EITHER     decided when the kernel starts, from the word the scan launch in front of it left in *p.iv_bad:
//                   by interval (p.iv) if every row of the mask is one, else the values are added.  No hand-over
//                   launch behind the tiled kernel; head_dim <= 64 (the register budget of both forms in one kernel).
constexpr int PF32_INTERVALS = 0, PF32_BIAS = 1, PF32_EITHER = 2;

template <typename T, int D, int S, int MODE>
__global__ __launch_bounds__(64 * PF32_WAVES, 2) void prefill_f32_kernel(AttnParams p, int nqb) {
    constexpr bool BIAS = MODE != PF32_INTERVALS;  // the mask-adding code is in the kernel
    constexpr int WPG = PF32_WAVES / S;   // wavefronts per key-split group
    constexpr int BM = 32 * WPG;          // query rows per workgroup
    // Which head dims a 32-row block of O^T holds.  With 2 or 4 blocks, row i of block db is dim NDB i + db: the
    // V operands of all blocks for one key then sit side by side and one 8- or 16-byte LDS read feeds NDB matrix
    // instructions (a 4-byte read per instruction leaves a lone wavefront waiting on LDS latency most of the time).
    constexpr int NDB = D / 32;
    constexpr bool PACKED = (NDB == 2 || NDB == 4);
    auto dim_of = [](int db, int i) __attribute__((always_inline)) { return PACKED ? NDB * i + db : 32 * db + i; };
    constexpr int KP = D * 4 + 16;  // row pitch in bytes: rows 4 banks apart -> conflict-free b128 reads
    constexpr int K_BYTES = PF32_BN * KP;
    constexpr int CPR = D / 4;      // 16-byte chunks per row
    constexpr int GT = 64 * WPG;    // threads of a group
    constexpr int NCH = PF32_BN * CPR / GT;
    static_assert(PF32_BN * CPR % GT == 0, "a group's threads must cover a tile evenly");
    // SOLO: a group is a single wavefront and the tile is too wide to stage K and V in registers at the same
    // time.  The wavefront then moves its tiles alone: K and V take turns in one register set and one LDS
    // buffer (V is fetched during S^T, the next K during P.V), and the loop needs no workgroup barrier.
    constexpr bool SOLO = (WPG == 1 && D > 64);
    static_assert(!(SOLO && BIAS), "the bias registers leave no room for this form");
    constexpr int G_BYTES = SOLO ? K_BYTES : 2 * K_BYTES;  // a group's tile buffers
    __shared__ __attribute__((aligned(16))) char smem[S * G_BYTES];
    auto lds_base = (__attribute__((address_space(3))) char *)smem;

    if constexpr (MODE == PF32_BIAS) {
        if (p.only_if_bad && *p.only_if_bad != p.bad_tag) return;  // the interval form of the mask has served the call
    } else if constexpr (MODE == PF32_INTERVALS) {
        if (p.iv_bad && *p.iv_bad == p.bad_tag) return;  // the mask is not made of intervals: the BIAS form takes the call
    }
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int ln = lane & 31;
    const int h2 = lane >> 5;
    const int grp = wave / WPG;     // key-split group
    const int wig = wave % WPG;     // wavefront inside the group: which 32 rows
    const int gtid = tid % GT;      // thread inside the group
    const int gbase = grp * G_BYTES;

    const int bh_count = p.B * p.H;
    const int nks = max(p.pf_nsplit, 1);
    const int ksplit = blockIdx.x % nks;  // which share of the keys (0 when the keys are not split over workgroups)
    const int id = snake_order(blockIdx.x / nks, gridDim.x / nks, p.snake_cus);
    const int qb = nqb - 1 - id / bh_count;
    int rem = id % bh_count;
    const int b = rem / p.H;
    int h = rem % p.H;
    if ((p.H & 7) == 0) h = (h & 7) * (p.H >> 3) + (h >> 3);
    const int g = h / p.G;
    // Rows of a tile beyond the sequence's own keys (kv_lens below the view's length: a ragged batch in one cache
    // allocation) are never fetched: what such rows hold, NaN included, must not reach the result as 0 x NaN in P . V.
    // (likewise the rows behind the last query's own position when the call says where its rows stand inside a longer
    // cache view: a causal descriptor with q_pos_offset + Sq below the view's length)
    int key_end = p.kv_lens ? min(p.Skv, max(p.kv_lens[b], 1)) : p.Skv;
    if (p.analytic && p.causal) key_end = (int)min((int64_t)key_end, max(p.q_pos_offset + p.Sq, (int64_t)1));

    const int q0 = qb * BM;
    const int qw0 = q0 + 32 * wig;
    const int query = qw0 + ln;
    // Q operand: Q[query][8 kc + 4 h2 .. +4]; requested before the bounds, whose table reads (mask tensors) would
    // otherwise delay these loads by a memory latency
    float4_t qreg[D / 8];
    {
        const int qrow = min(query, p.Sq - 1);
        const T *qp = (const T *)p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)qrow * p.qs[2];
#pragma unroll
        for (int kc = 0; kc < D / 8; kc++)
            qreg[kc] = 8 * kc + 4 * h2 < p.D ? load4(qp + 8 * kc + 4 * h2) : float4_t{0.f, 0.f, 0.f, 0.f};
    }
    // uniform over the launch
    const bool bias_on = MODE == PF32_BIAS || (MODE == PF32_EITHER && *p.iv_bad == p.bad_tag);
    RowBounds rb = row_bounds(p, MODE == PF32_BIAS ? nullptr : p.iv, b, q0, BM, qw0, lane);
    if constexpr (MODE == PF32_EITHER) {
        // the table was read whatever the scan found (its loads need not wait for that word); without the interval
        // form the bounds are those of a call whose mask is added
        if (bias_on) rb = row_bounds(p, nullptr, b, q0, BM, qw0, lane);
    }
    if (nks > 1) {  // this workgroup's share of the keys
        const int c_lo = ksplit * p.pf_chunk, c_hi = c_lo + p.pf_chunk;
        rb.lo_wg = max(rb.lo_wg, c_lo), rb.hi_wg = min(rb.hi_wg, c_hi);
        rb.lo_w = max(rb.lo_w, c_lo), rb.hi_w = min(rb.hi_w, c_hi);
        rb.full_lo_w = max(rb.full_lo_w, c_lo), rb.full_hi_w = min(rb.full_hi_w, c_hi);
        rb.klo = max(rb.klo, c_lo), rb.khi = min(rb.khi, c_hi);
    }
    const int lo_wg = rb.lo_wg, hi_wg = rb.hi_wg, lo_w = rb.lo_w, hi_w = rb.hi_w;
    const bool wave_has_rows = qw0 < p.Sq;

    const T *kg = (const T *)p.k + b * p.ks[0] + g * p.ks[1];
    const T *vg = (const T *)p.v + b * p.vs[0] + g * p.vs[1];

    float16_t o[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    // scores reach the softmax in the base-2 domain: raw dot products times scale * log2(e); with BIAS they are
    // scaled, biased, and then only multiplied by log2(e)
    const float scale2 = bias_on ? PF32_LOG2E : p.scale * PF32_LOG2E;
    const T *mrow = nullptr;
    if constexpr (BIAS)
        mrow = (const T *)p.mask + (int64_t)(p.mask_kind == FHIP_MASK_QK ? min(query, p.Sq - 1) : b) * p.ms0;

    const int j_begin = (lo_wg / PF32_BN) * PF32_BN;
    const int ntiles = hi_wg > j_begin ? (hi_wg - j_begin + PF32_BN - 1) / PF32_BN : 0;
    // a thread's chunks of a tile are a fixed number of rows apart when its group's threads cover whole rows
    constexpr bool AFFINE = (GT % CPR == 0);
    constexpr int RSTEP = AFFINE ? GT / CPR : 0;
    const bool whole_rows = p.D == D;

    // One tile's math: S^T from the K image at the start of the group's buffer, online softmax, then `between`
    // (how the single-wavefront form swaps V into the buffer), then O^T += V^T . P^T from the V image at `voff`.
    auto tile_math = [&](int j0, int voff, auto &&between) __attribute__((always_inline)) {
        float bias[BIAS ? 16 : 1];
        if constexpr (BIAS) {  // requested before the matrix work that hides their latency
            if (bias_on) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int key = j0 + 8 * (r >> 2) + 4 * h2 + (r & 3);
                    bias[r] = key < p.Skv ? to_float(mrow[(int64_t)key * p.ms1]) : 0.0f;
                }
            }
        }

        // S^T: contraction step (kc, i) uses dim 8 kc + 4 h2 + i on both operands
        float16_t s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.0f;
#pragma unroll
        for (int kc = 0; kc < D / 8; kc++) {
            const float4_t a = *LDS32_PTR(float4_t, gbase + ln * KP + (8 * kc + 4 * h2) * 4);
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

        if constexpr (BIAS) {
            if (bias_on) {
#pragma unroll
                for (int r = 0; r < 16; r++) s[r] = s[r] * p.scale + bias[r];
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

        between();

        // O^T += V^T . P^T: contraction step r pairs this half-wave's key 8 (r/4) + 4 h2 + r%4
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int krow = 8 * (r >> 2) + 4 * h2 + (r & 3);
            if constexpr (NDB == 4) {
                const float4_t a = *LDS32_PTR(float4_t, gbase + voff + krow * KP + ln * 16);
#pragma unroll
                for (int db = 0; db < 4; db++) o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[db], s[r], o[db], 0, 0, 0);
            } else if constexpr (NDB == 2) {
                typedef float float2_t __attribute__((ext_vector_type(2)));
                const float2_t a = *LDS32_PTR(float2_t, gbase + voff + krow * KP + ln * 8);
#pragma unroll
                for (int db = 0; db < 2; db++) o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[db], s[r], o[db], 0, 0, 0);
            } else {
#pragma unroll
                for (int db = 0; db < NDB; db++) {
                    const float a = *LDS32_PTR(float, gbase + voff + krow * KP + (32 * db + ln) * 4);
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, s[r], o[db], 0, 0, 0);
                }
            }
        }
    };

    if constexpr (SOLO) {
        // this wavefront's own tiles: those of its group (t % S == grp) among the tiles its rows see
        int ta = 0, tb = 0;
        if (wave_has_rows && hi_w > lo_w) {
            ta = (lo_w - j_begin) / PF32_BN;
            tb = min(ntiles, (hi_w - j_begin + PF32_BN - 1) / PF32_BN);
        }
        float4_t st[NCH];
        auto load_rows = [&](const T *base, int64_t stride, int j0) __attribute__((always_inline)) {
            if (AFFINE && whole_rows && j0 + PF32_BN <= key_end) {
                // a tile inside the key axis with rows as wide as the kernel's: one address per thread, the
                // chunks a fixed number of rows apart, no clamp and no branch per chunk
                const T *p0 = base + (int64_t)(j0 + lane / CPR) * stride + (lane % CPR) * 4;
                const int64_t step = (int64_t)RSTEP * stride;
#pragma unroll
                for (int i = 0; i < NCH; i++) st[i] = load4(p0 + i * step);
                return;
            }
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                const int cid = lane + 64 * i;
                const int row = cid / CPR, col = cid % CPR;
                const int key = min(j0 + row, key_end - 1);
                st[i] = col * 4 < p.D ? load4(base + (int64_t)key * stride + col * 4) : float4_t{0.f, 0.f, 0.f, 0.f};
            }
        };
        auto store_rows = [&]() __attribute__((always_inline)) {
            wave_lds_sync();  // the reads of the image being replaced are done
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                const int cid = lane + 64 * i;
                *LDS32_PTR(float4_t, gbase + (cid / CPR) * KP + (cid % CPR) * 16) = st[i];
            }
            wave_lds_sync();
        };
        int t = ta + ((grp - ta) % S + S) % S;
        if (t < tb) load_rows(kg, p.ks[2], j_begin + t * PF32_BN);
        for (; t < tb; t += S) {
            const int j0 = j_begin + t * PF32_BN;
            store_rows();                  // K(t)
            load_rows(vg, p.vs[2], j0);    // V(t) arrives during S^T
            tile_math(j0, 0, [&]() __attribute__((always_inline)) {
                store_rows();              // V(t) replaces K(t)
                if (t + S < tb) load_rows(kg, p.ks[2], j0 + S * PF32_BN);  // K of the next tile arrives during P.V
            });
        }
    } else {
        float4_t kst[NCH], vst[NCH];
        auto load_tile = [&](int j0) {
            if (AFFINE && whole_rows && j0 + PF32_BN <= key_end) {  // see load_rows above
                const T *pk = kg + (int64_t)(j0 + gtid / CPR) * p.ks[2] + (gtid % CPR) * 4;
                const T *pv = vg + (int64_t)(j0 + gtid / CPR) * p.vs[2] + (gtid % CPR) * 4;
                const int64_t kstep = (int64_t)RSTEP * p.ks[2], vstep = (int64_t)RSTEP * p.vs[2];
#pragma unroll
                for (int i = 0; i < NCH; i++) {
                    kst[i] = load4(pk + i * kstep);
                    vst[i] = load4(pv + i * vstep);
                }
                return;
            }
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                const int cid = gtid + GT * i;
                const int row = cid / CPR, col = cid % CPR;
                const int key = min(j0 + row, key_end - 1);
                const bool in_row = col * 4 < p.D;  // a head_dim below D is padded with zeros
                kst[i] = in_row ? load4(kg + (int64_t)key * p.ks[2] + col * 4) : float4_t{0.f, 0.f, 0.f, 0.f};
                vst[i] = in_row ? load4(vg + (int64_t)key * p.vs[2] + col * 4) : float4_t{0.f, 0.f, 0.f, 0.f};
            }
        };
        auto store_tile = [&]() {
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                const int cid = gtid + GT * i;
                const int row = cid / CPR, col = cid % CPR;
                *LDS32_PTR(float4_t, gbase + row * KP + col * 16) = kst[i];
                *LDS32_PTR(float4_t, gbase + K_BYTES + row * KP + col * 16) = vst[i];
            }
        };

        // group g takes the tiles j_begin + (it * S + g) * 32; every group runs the same number of iterations
        // (the barriers are workgroup-wide), a group without a tile in the last one idles through it
        const int niter = (ntiles + S - 1) / S;
        if (grp < ntiles) load_tile(j_begin + grp * PF32_BN);

        for (int it = 0; it < niter; it++) {
            const int t = it * S + grp;
            const int j0 = j_begin + t * PF32_BN;
            const bool have = t < ntiles;
            lds_barrier();  // everyone finished reading the previous tile (LDS-only barrier: the prefetch
            if (have) store_tile();  // issued below stays in flight across the math)
            lds_barrier();
            if (t + S < ntiles) load_tile(j0 + S * PF32_BN);

            const bool tile_visible = have && wave_has_rows && j0 < hi_w && j0 + PF32_BN > lo_w;
            if (!tile_visible) continue;
            tile_math(j0, K_BYTES, []() {});
        }
    }

    if constexpr (S > 1) {
        // merge the groups: groups 1.. park (m, l, O) in LDS, one value per lane and register, group 0
        // folds them into its own state (log-sum-exp merge, as the split-KV combine does)
        constexpr int NR = 16 * (D / 32) + 2;            // registers per lane
        static_assert((S - 1) * WPG * NR * 256 <= S * G_BYTES, "merge staging exceeds the tile buffers");
        lds_barrier();  // the tile buffers are free
        if (grp > 0) {
            const int slot = ((grp - 1) * WPG + wig) * NR * 256 + lane * 4;
#pragma unroll
            for (int db = 0; db < D / 32; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) *LDS32_PTR(float, slot + (16 * db + r) * 256) = o[db][r];
            *LDS32_PTR(float, slot + (NR - 2) * 256) = m;
            *LDS32_PTR(float, slot + (NR - 1) * 256) = l;
        }
        lds_barrier();
        if (grp > 0) return;
#pragma unroll
        for (int gsrc = 1; gsrc < S; gsrc++) {
            const int slot = ((gsrc - 1) * WPG + wig) * NR * 256 + lane * 4;
            const float m_other = *LDS32_PTR(float, slot + (NR - 2) * 256);
            const float l_other = *LDS32_PTR(float, slot + (NR - 1) * 256);
            const float m_all = fmaxf(m, m_other);
            const float m_safe = (m_all == -INFINITY) ? 0.0f : m_all;
            const float wa = __builtin_amdgcn_exp2f(m - m_safe), wb = __builtin_amdgcn_exp2f(m_other - m_safe);
            l = l * wa + l_other * wb;
#pragma unroll
            for (int db = 0; db < D / 32; db++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    o[db][r] = o[db][r] * wa + *LDS32_PTR(float, slot + (16 * db + r) * 256) * wb;
            m = m_all;
        }
    }
    const float l_tot = half_swap_sum32(l);
    if (nks > 1) {
        // park this share's state; the merge kernel normalises
        if (query < p.Sq) {
            float *ws = p.partials + ((((int64_t)b * p.H + h) * p.Sq + query) * nks + ksplit) * p.pf_pitch;
#pragma unroll
            for (int db = 0; db < D / 32; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int dim = dim_of(db, 8 * (r >> 2) + 4 * h2 + (r & 3));
                    if (dim < p.D) ws[dim] = o[db][r];
                }
            if (h2 == 0) {
                ws[p.D] = m;
                ws[p.D + 1] = l_tot;
            }
        }
        return;
    }
    if (query < p.Sq) {
        const int64_t ob = b * p.os[0] + h * p.os[1] + (int64_t)query * p.os[2];
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int dim = dim_of(db, 8 * (r >> 2) + 4 * h2 + (r & 3));
                if (dim < p.D) store_out<T>(p, ob + dim * p.os[3], o[db][r] / l_tot);  // no visible key: 0/0 = NaN like the reference
            }
    }
}

// Merge of the key shares: one wavefront per (batch, head, query row), log-sum-exp over the shares (the state is
// in the base-2 domain), then the division the single-pass form does in its epilogue.
template <typename T>
__global__ __launch_bounds__(256) void prefill_f32_merge_kernel(AttnParams p) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int64_t rows = (int64_t)p.B * p.H * p.Sq;
    if (row >= rows) return;
    // the same hand-over between the interval form and the mask-adding form as in the main kernel (none when the
    // main kernel held both forms)
    if (!p.iv_either && ((p.iv_bad && *p.iv_bad == p.bad_tag) || (p.only_if_bad && *p.only_if_bad != p.bad_tag))) return;
    const int query = (int)(row % p.Sq);
    const int h = (int)((row / p.Sq) % p.H), b = (int)(row / p.Sq / p.H);
    const int D = p.D, ns = p.pf_nsplit, pitch = p.pf_pitch;
    const float *ws = p.partials + row * ns * pitch;
    // eight shares per round of loads (a round costs one memory latency)
    float M = -INFINITY, L = 0.0f, A[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // dims lane, lane + 64, lane + 128, lane + 192
    for (int s0 = 0; s0 < ns; s0 += 8) {
        float ms[8], ls[8], av[8][4];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const bool ok = s0 + u < ns;
            const float *src = ws + (ok ? s0 + u : s0) * pitch;
            ms[u] = ok ? src[D] : -INFINITY;
            ls[u] = ok ? src[D + 1] : 0.0f;
#pragma unroll
            for (int k = 0; k < 4; k++) av[u][k] = (ok && lane + 64 * k < D) ? src[lane + 64 * k] : 0.0f;
        }
        float Mn = M;
#pragma unroll
        for (int u = 0; u < 8; u++) Mn = fmaxf(Mn, ms[u]);
        const float Ms = (Mn == -INFINITY) ? 0.0f : Mn;
        const float c = __builtin_amdgcn_exp2f(M - Ms);
        L *= c;
#pragma unroll
        for (int k = 0; k < 4; k++) A[k] *= c;
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const float w = __builtin_amdgcn_exp2f(ms[u] - Ms);
            L += w * ls[u];
#pragma unroll
            for (int k = 0; k < 4; k++) A[k] += w * av[u][k];
        }
        M = Mn;
    }
    const int64_t ob = b * p.os[0] + h * p.os[1] + (int64_t)query * p.os[2];
#pragma unroll
    for (int k = 0; k < 4; k++)
        if (lane + 64 * k < D) store_out<T>(p, ob + (lane + 64 * k) * p.os[3], A[k] / L);  // no visible key: 0/0 = NaN
}

// ---- head_dim 129 .. 256 (Gemma-3's key length is 256) -------------------------------------------------------
// A wavefront cannot hold 256 dims of Q and O for 32 rows, so two wavefronts share the 32 rows: wavefront
// `hf` of the pair owns dims [128 hf, 128 hf + 128) of Q, K, V and O.  Per key tile each computes its half of
// the contraction S^T = K Q^T, the halves are exchanged through LDS (in the K tile's space, which is free by
// then) and added, both run the same softmax on the same sums, and each accumulates its half of O^T.
// Workgroup = 2 pairs = 64 query rows; K, V tiles of 32 keys x 256 dims (zero-padded above head_dim).
constexpr int PFW_DP = 256, PFW_DH = 128;

template <typename T>
__global__ __launch_bounds__(64 * PF32_WAVES, 2) void prefill_f32_wide_kernel(AttnParams p, int nqb) {
    constexpr int BM = 64;
    constexpr int KP = PFW_DP * 4 + 16;
    constexpr int K_BYTES = PF32_BN * KP;
    constexpr int CPR = PFW_DP / 4;
    constexpr int NCH = PF32_BN * CPR / (64 * PF32_WAVES);
    static_assert(PF32_WAVES * 16 * 256 <= K_BYTES, "the score exchange must fit the K tile's space");
    __shared__ __attribute__((aligned(16))) char smem[2 * K_BYTES];
    auto lds_base = (__attribute__((address_space(3))) char *)smem;

    if (p.iv_bad && *p.iv_bad == p.bad_tag) return;  // the mask is not made of intervals: the general kernel takes the call
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int ln = lane & 31;
    const int h2 = lane >> 5;
    const int pr = wave >> 1;  // which 32 rows
    const int hf = wave & 1;   // which half of the dims
    const int d0 = PFW_DH * hf;

    // Packed form (at most 32 query rows, an even GQA group): the two pairs hold rows 0..31 of two query heads that share
    // a KV head, so both work on every tile the workgroup moves (with one head per workgroup the second pair has no
    // rows) and a few new rows on a long cache need half the workgroups.
    const int pack = p.pf_pack;
    const int heads = pack ? p.H / 2 : p.H;  // head units per batch entry
    const int bh_count = p.B * heads;
    const int nks = max(p.pf_nsplit, 1);
    const int ksplit = blockIdx.x % nks;  // which share of the keys (0 when the keys are not split over workgroups)
    const int id = snake_order(blockIdx.x / nks, gridDim.x / nks, p.snake_cus);
    const int qb = nqb - 1 - id / bh_count;
    int rem = id % bh_count;
    const int b = rem / heads;
    int h = rem % heads;
    if (pack) h = 2 * h + pr;
    else if ((p.H & 7) == 0) h = (h & 7) * (p.H >> 3) + (h >> 3);
    const int g = h / p.G;
    // Rows of a tile beyond the sequence's own keys (kv_lens below the view's length: a ragged batch in one cache
    // allocation) are never fetched: what such rows hold, NaN included, must not reach the result as 0 x NaN in P . V.
    // (likewise the rows behind the last query's own position when the call says where its rows stand inside a longer
    // cache view: a causal descriptor with q_pos_offset + Sq below the view's length)
    int key_end = p.kv_lens ? min(p.Skv, max(p.kv_lens[b], 1)) : p.Skv;
    if (p.analytic && p.causal) key_end = (int)min((int64_t)key_end, max(p.q_pos_offset + p.Sq, (int64_t)1));

    const int q0 = pack ? 0 : qb * BM;
    const int qw0 = pack ? 0 : q0 + 32 * pr;
    const int query = qw0 + ln;
    RowBounds rb = row_bounds(p, b, q0, pack ? 32 : BM, qw0, lane);
    if (nks > 1) {  // this workgroup's share of the keys
        const int c_lo = ksplit * p.pf_chunk, c_hi = c_lo + p.pf_chunk;
        rb.lo_wg = max(rb.lo_wg, c_lo), rb.hi_wg = min(rb.hi_wg, c_hi);
        rb.lo_w = max(rb.lo_w, c_lo), rb.hi_w = min(rb.hi_w, c_hi);
        rb.full_lo_w = max(rb.full_lo_w, c_lo), rb.full_hi_w = min(rb.full_hi_w, c_hi);
        rb.klo = max(rb.klo, c_lo), rb.khi = min(rb.khi, c_hi);
    }
    const int lo_wg = rb.lo_wg, hi_wg = rb.hi_wg, lo_w = rb.lo_w, hi_w = rb.hi_w;
    const bool wave_has_rows = qw0 < p.Sq;

    float4_t qreg[PFW_DH / 8];
    {
        const int qrow = min(query, p.Sq - 1);
        const T *qp = (const T *)p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)qrow * p.qs[2];
#pragma unroll
        for (int kc = 0; kc < PFW_DH / 8; kc++) {
            const int dim = d0 + 8 * kc + 4 * h2;
            qreg[kc] = dim < p.D ? load4(qp + dim) : float4_t{0.f, 0.f, 0.f, 0.f};
        }
    }
    const T *kg = (const T *)p.k + b * p.ks[0] + g * p.ks[1];
    const T *vg = (const T *)p.v + b * p.vs[0] + g * p.vs[1];

    float16_t o[PFW_DH / 32];
#pragma unroll
    for (int db = 0; db < PFW_DH / 32; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    const float scale2 = p.scale * PF32_LOG2E;

    // K and V take turns in one set of staging registers: V(j) is in flight while K(j) is multiplied, K(j+1)
    // while V(j) is
    float4_t st[NCH];
    auto load_rows = [&](const T *base, const int64_t row_stride, int j0) {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int cid = tid + 64 * PF32_WAVES * i;
            const int row = cid / CPR, col = cid % CPR;
            const int key = min(j0 + row, key_end - 1);
            st[i] = col * 4 < p.D ? load4(base + (int64_t)key * row_stride + col * 4) : float4_t{0.f, 0.f, 0.f, 0.f};
        }
    };
    auto store_rows = [&](int lds_off) {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int cid = tid + 64 * PF32_WAVES * i;
            const int row = cid / CPR, col = cid % CPR;
            *LDS32_PTR(float4_t, lds_off + row * KP + col * 16) = st[i];
        }
    };

    const int j_begin = (lo_wg / PF32_BN) * PF32_BN;
    if (j_begin < hi_wg) load_rows(kg, p.ks[2], j_begin);

    // every wavefront passes the same four barriers per tile, whether or not its rows see the tile
    for (int j0 = j_begin; j0 < hi_wg; j0 += PF32_BN) {
        store_rows(0);                    // K(j); its space is free since the last barrier of the previous tile
        load_rows(vg, p.vs[2], j0);       // V(j), needed after the softmax
        lds_barrier();
        const bool tile_visible = wave_has_rows && j0 < hi_w && j0 + PF32_BN > lo_w;  // the same for both halves

        // this half of S^T: contraction step (kc, i) uses dim d0 + 8 kc + 4 h2 + i on both operands
        float16_t s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.0f;
        if (tile_visible) {
#pragma unroll
            for (int kc = 0; kc < PFW_DH / 8; kc++) {
                const float4_t a = *LDS32_PTR(float4_t, ln * KP + (d0 + 8 * kc + 4 * h2) * 4);
#pragma unroll
                for (int i = 0; i < 4; i++) s = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], qreg[kc][i], s, 0, 0, 0);
            }
        }
        lds_barrier();  // the K tile has been read: its space takes the exchange
        if (tile_visible) {
#pragma unroll
            for (int r = 0; r < 16; r++) *LDS32_PTR(float, wave * 4096 + r * 256 + lane * 4) = s[r];
        }
        lds_barrier();
        if (tile_visible) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float other = *LDS32_PTR(float, (wave ^ 1) * 4096 + r * 256 + lane * 4);
                s[r] = hf == 0 ? s[r] + other : other + s[r];  // low + high half on both wavefronts: identical sums
            }
        }
        store_rows(K_BYTES);              // V(j); every wavefront is past P.V of the previous tile
        if (j0 + PF32_BN < hi_wg) load_rows(kg, p.ks[2], j0 + PF32_BN);  // K(j+1)
        lds_barrier();                    // V(j) visible, the exchange has been read
        if (!tile_visible) continue;

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
        for (int db = 0; db < PFW_DH / 32; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[db][r] *= corr;

        // this half of O^T += V^T . P^T
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int krow = 8 * (r >> 2) + 4 * h2 + (r & 3);
#pragma unroll
            for (int db = 0; db < PFW_DH / 32; db++) {
                const float a = *LDS32_PTR(float, K_BYTES + krow * KP + (d0 + 32 * db + ln) * 4);
                o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, s[r], o[db], 0, 0, 0);
            }
        }
    }

    const float l_tot = half_swap_sum32(l);
    if (nks > 1) {
        // park this share's state (each wavefront of the pair its half of the dims); the merge kernel normalises
        if (query < p.Sq) {
            float *ws = p.partials + ((((int64_t)b * p.H + h) * p.Sq + query) * nks + ksplit) * p.pf_pitch;
#pragma unroll
            for (int db = 0; db < PFW_DH / 32; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int dim = d0 + 32 * db + 8 * (r >> 2) + 4 * h2 + (r & 3);
                    if (dim < p.D) ws[dim] = o[db][r];
                }
            if (hf == 0 && h2 == 0) {
                ws[p.D] = m;
                ws[p.D + 1] = l_tot;
            }
        }
        return;
    }
    if (query < p.Sq) {
        const int64_t ob = b * p.os[0] + h * p.os[1] + (int64_t)query * p.os[2];
#pragma unroll
        for (int db = 0; db < PFW_DH / 32; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int dim = d0 + 32 * db + 8 * (r >> 2) + 4 * h2 + (r & 3);
                if (dim < p.D) store_out<T>(p, ob + dim * p.os[3], o[db][r] / l_tot);  // no visible key: 0/0 = NaN like the reference
            }
    }
}

template <typename T>
static int launch_merge_t(const AttnParams &p, hipStream_t stream);

// query heads that share one workgroup of the wide-head kernel (0: one head, up to 64 rows)
static int prefill_f32_wide_pack(int G, int Sq, int D) { return (D > 128 && Sq <= 32 && G >= 2 && G % 2 == 0) ? 2 : 0; }

template <typename T>
static int launch_wide(const AttnParams &p_in, hipStream_t stream) {
    if (p_in.mask && !p_in.iv) {
        set_error("prefill f32: a mask tensor without its interval form is not supported above head_dim 128");
        return FHIP_ERR_UNSUPPORTED;
    }
    AttnParams p = p_in;
    p.pf_pack = prefill_f32_wide_pack(p.G, p.Sq, p.D);
    const int nqb = p.pf_pack ? 1 : (p.Sq + 63) / 64;
    const long blocks = (long)nqb * p.B * (p.pf_pack ? p.H / 2 : p.H) * (p.pf_nsplit > 1 ? p.pf_nsplit : 1);
    if (blocks > 0x7fffffffL) {
        set_error("prefill f32: too many workgroups (%ld)", blocks);
        return FHIP_ERR_UNSUPPORTED;
    }
    FHIP_LAUNCH_MAIN(prefill_f32_wide_kernel<T>, dim3((unsigned)blocks), dim3(64 * PF32_WAVES), stream, p, p, nqb);
    FHIP_HIP_CHECK(hipGetLastError());
    if (p.pf_nsplit > 1) return launch_merge_t<T>(p, stream);
    return FHIP_OK;
}

template <typename T>
static int launch_merge_t(const AttnParams &p, hipStream_t stream) {
    const int64_t rows = (int64_t)p.B * p.H * p.Sq;
    hipLaunchKernelGGL(prefill_f32_merge_kernel<T>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, p);
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

int launch_prefill_merge(const AttnParams &p, fhip_dtype dtype, hipStream_t stream) {
    if (dtype == FHIP_F16) return launch_merge_t<half_t>(p, stream);
    if (dtype == FHIP_BF16) return launch_merge_t<bf16_t>(p, stream);
    return launch_merge_t<float>(p, stream);
}

template <typename T, int S, int MODE>
static int launch_split(const AttnParams &p, hipStream_t stream) {
    constexpr bool BIAS = MODE != PF32_INTERVALS;
    constexpr int BM = 32 * (PF32_WAVES / S);
    const int nqb = (p.Sq + BM - 1) / BM;
    const long blocks = (long)nqb * p.B * p.H * (p.pf_nsplit > 1 ? p.pf_nsplit : 1);
    if (blocks > 0x7fffffffL) {
        set_error("prefill f32: too many workgroups (%ld)", blocks);
        return FHIP_ERR_UNSUPPORTED;
    }
    dim3 grid((unsigned)blocks), block(64 * PF32_WAVES);
    switch ((p.D + 31) / 32 * 32) {  // the kernel's D is head_dim rounded up to a multiple of 32
        case 32: FHIP_LAUNCH_MAIN((prefill_f32_kernel<T, 32, S, MODE>), grid, block, stream, p, p, nqb); break;
        case 64: FHIP_LAUNCH_MAIN((prefill_f32_kernel<T, 64, S, MODE>), grid, block, stream, p, p, nqb); break;
        case 96:
            if constexpr (S <= (BIAS ? 1 : 4) && MODE != PF32_EITHER)
                FHIP_LAUNCH_MAIN((prefill_f32_kernel<T, 96, S, MODE>), grid, block, stream, p, p, nqb);
            break;
        case 128:
            if constexpr (S <= (BIAS ? 1 : 4) && MODE != PF32_EITHER)
                FHIP_LAUNCH_MAIN((prefill_f32_kernel<T, 128, S, MODE>), grid, block, stream, p, p, nqb);
            break;
        default: set_error("prefill f32 kernel: head_dim %d is not a multiple of 4 up to 128", p.D); return FHIP_ERR_UNSUPPORTED;
    }
    FHIP_HIP_CHECK(hipGetLastError());
    if (p.pf_nsplit > 1) return launch_merge_t<T>(p, stream);
    return FHIP_OK;
}

// Few query rows on a long cache (a new chat turn, a prompt fed in pieces): the grid of query blocks alone leaves
// most CUs idle, so the keys are split over workgroups as well, down to 512 keys per share, until there are about
// two workgroups per CU.  Square causal calls are left alone (their shares would be uneven, and they fill the
// chip from 1024 rows on).
void prefill_f32_plan(int B, int H, int G, int Sq, int Skv, int D, bool causal_square, int compute_units, int *nsplit, int *chunk) {
    *nsplit = 1;
    *chunk = Skv;
    if (causal_square) return;
    const int bm = D > 128 ? 64 : 32;  // the finest query blocking the kernel has
    const int pack = prefill_f32_wide_pack(G, Sq, D);
    const long wgs = pack ? (long)B * (H / 2) : (long)B * H * ((Sq + bm - 1) / bm);
    if (wgs > compute_units) return;  // the query blocks alone keep at least half the chip busy (two workgroups per CU)
    const long want = (2L * compute_units + wgs - 1) / wgs;
    // Shares of at least 512 keys (256 in the packed form, which has half the workgroups); while that leaves CUs without
    // a workgroup, down to 256 and then 128 keys: a workgroup alone on its CU spends most of a tile waiting for the
    // tile's rows (~7 us per 32-key tile in the wide-head kernel, ~2 us below), so more, shorter workgroups win until
    // the chip is full (f32, B1: head_dim 256, 2048 keys, 9 rows 55 -> 36 us; head_dim 128, 2048 keys, 20 rows 34 -> 26,
    // 1024 keys 33 -> 21).  Shorter shares than needed merge too often (head_dim 256, B1 x 8192 keys, 32 rows: 84 us with
    // 256 shares of 8 tiles, 101 us with 512 of 4).
    long most = Skv / (pack ? 256 : 512);
    // (only for calls that are clearly a few rows on a longer cache: a square prompt masked by a tensor keeps the plan
    // of its analytic twin, and with it the same bits)
    const bool few_rows = 2L * Sq <= Skv;
    if (few_rows && (want < most ? want : most) * wgs < compute_units) most = Skv / 256;
    if (few_rows && (want < most ? want : most) * wgs < compute_units) most = Skv / 128;
    long ns = want < most ? want : most;
    if (ns < 2) return;
    long c = (Skv + ns - 1) / ns;
    c = (c + 31) / 32 * 32;
    *chunk = (int)c;
    *nsplit = (int)((Skv + c - 1) / c);
}

size_t prefill_f32_workspace_bytes(int B, int H, int Sq, int D, int nsplit) {
    if (nsplit <= 1) return 0;
    return (size_t)B * H * Sq * nsplit * (size_t)(D + 2) * sizeof(float);
}

// 16-bit tensors are served by the unsplit forms only (their own matrix-core kernel takes the common shapes)
template <typename T>
static int launch_prefill_f32_t(const AttnParams &p, hipStream_t stream) {
    if (p.D > 128) return launch_wide<T>(p, stream);
    // Split the keys of a query block over 2 or 4 wavefront groups while the unsplit grid is only a few
    // workgroups per CU: the longest (last causal) query block then sets the run time, and halving it pays
    // even when every CU has work.  Measured break-even: about 4 workgroups per CU at head_dim <= 64, 2 above
    // (the bigger tiles leave less to gain).  Four groups: below two 64-row workgroups per CU at head_dim <= 64;
    // above, where each wavefront moves its tiles alone, up to one per CU.
    const int cus = p.cus > 0 ? p.cus : 256;
    const long bh = (long)p.B * p.H * (p.pf_nsplit > 1 ? p.pf_nsplit : 1);
    const long wg1 = bh * ((p.Sq + 127) / 128), wg2 = bh * ((p.Sq + 63) / 64);
    const bool small_dim = p.D <= 64;
    int split = 1;
    if (wg1 <= (small_dim ? 4L : 2L) * cus) split = 2;
    if (split == 2 && (small_dim ? wg2 < 2L * cus : (wg2 < cus || (wg2 == cus && p.Skv >= 256)))) split = 4;
    // the last 64-row block at least half empty (96 rows: 128 computed; 32 rows: 64): 32-row blocks compute only what
    // is there (f32, 32/8 heads, head_dim 128, 8192 keys: 96 rows 221 -> 180 us at batch 1, 1252 -> 1005 at batch 8; 32
    // rows at batch 8 545 -> 387 us)
    if (split == 2 && !small_dim && (p.Sq + 31) / 32 * 32 < (p.Sq + 63) / 64 * 64 && bh * ((p.Sq + 31) / 32) <= 4L * cus) split = 4;
    if (sizeof(T) != 4) split = 1;
    // a mask tensor without its interval form is added element by element (the 16 bias registers leave no
    // room for the key-split form at head_dim 96 / 128)
    const bool either = p.mask && p.iv && p.iv_either;  // the kernel reads the scan's verdict itself
    if (either && !small_dim) {
        set_error("internal: the two-form f32 kernel takes head_dim <= 64");
        return FHIP_ERR_UNSUPPORTED;
    }
    const bool add_mask = p.mask && !p.iv;
    if (add_mask && !small_dim) split = 1;
    AttnParams ps = p;
    {
        const long blocks = bh * ((p.Sq + 128 / split - 1) / (128 / split));
        ps.snake_cus = (blocks > cus && blocks <= 2L * cus) ? cus : 0;
    }
    if (either) {
        if constexpr (sizeof(T) == 4) {
            if (split == 4) return launch_split<T, 4, PF32_EITHER>(ps, stream);
            if (split == 2) return launch_split<T, 2, PF32_EITHER>(ps, stream);
        }
        return launch_split<T, 1, PF32_EITHER>(ps, stream);
    }
    if (add_mask) {
        if constexpr (sizeof(T) == 4) {
            if (split == 4) return launch_split<T, 4, PF32_BIAS>(ps, stream);
            if (split == 2) return launch_split<T, 2, PF32_BIAS>(ps, stream);
        }
        return launch_split<T, 1, PF32_BIAS>(ps, stream);
    }
    if constexpr (sizeof(T) == 4) {
        if (split == 4) return launch_split<T, 4, PF32_INTERVALS>(ps, stream);
        if (split == 2) return launch_split<T, 2, PF32_INTERVALS>(ps, stream);
    }
    return launch_split<T, 1, PF32_INTERVALS>(ps, stream);
}

int launch_prefill_f32(const AttnParams &p, fhip_dtype dtype, hipStream_t stream) {
    if (dtype == FHIP_F16) return launch_prefill_f32_t<half_t>(p, stream);
    if (dtype == FHIP_BF16) return launch_prefill_f32_t<bf16_t>(p, stream);
    return launch_prefill_f32_t<float>(p, stream);
}

}  // namespace fhip
