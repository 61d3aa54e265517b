// Prefill attention for f16 / bf16 on the gfx950 matrix cores.
//
// Workgroup = 8 wavefronts = 256 query rows of one (batch, head); each wavefront owns 32 rows.
// Keys/values are walked in tiles of 64 rows that go from global memory straight into a three-stage
// LDS ring (direct-to-LDS buffer loads, no staging registers).  Per tile and wavefront:
//   S^T (64 keys x 32 queries)  = K_tile . Q^T      v_mfma_f32_32x32x16  (A = K from LDS, B = Q in registers)
//   Q is multiplied once by the power-of-two part of scale * log2(e) (exact); the rest, a factor rr in [1, 2),
//   multiplies the scores in f32: a probability is exp2(fma(s, rr, -m * rr)), one fused multiply-add and one
//   exponential per score, with m the row's reference exponent
//   online softmax down the key axis: with S^T every lane owns ONE query column and 16 keys of it per 32-key
//   block, so row sums are in-lane folds (the two half-rows are added once, at the end).  No maximum is taken
//   per tile: the reference m is the maximum the row had when it was last set, and it is moved (and l and O
//   rescaled) only when a lane's probabilities of a tile sum to more than 2^15, i.e. before one of them could
//   leave the 16-bit type's range; on random data that is the first tile and almost never again
//   O^T (D x 32 queries)       += V_tile^T . P^T    A = V^T read from row-major LDS with the
//   transposing LDS load ds_read_b64_tr_b16, B = P^T taken straight from the S^T accumulator
//   registers (the contraction index is permuted identically on both operands)
// The two wavefronts that share a SIMD (w and w + 4) run half a tile out of phase: while one is in
// its matrix phase (S^T of the current tile, then P.V of the previous one) the other is in its
// vector phase (softmax, tile loads), so the MFMA pipe and the VALU are busy at the same time.
// Phases are separated by workgroup barriers; the tile loads ride on the same barriers.  The vector
// phase uses no dot-product instructions: on this chip they queue behind the MFMAs of the other
// wavefront instead of running beside them.
// All accumulation is f32; P is rounded to the input type for the second product.
// Key-split form (template parameter KS): the workgroup owns 128 query rows and its two wavefront groups
// take alternate key tiles of the same rows, each through the same matrix / vector phases, and merge their
// (m, l, O) through LDS at the end: twice the workgroups, half the longest one, for grids that do not fill
// the chip (see use_key_split_form).
// Masking is by interval: every query row sees one range of keys, known analytically (causal with
// offset, sliding window, per-batch kv length, tail of the key axis) or read from the interval form
// of a dense mask tensor (attn_bounds.h, mask_intervals.hip); key tiles that are invisible to the
// whole workgroup are never loaded, and tiles fully visible to a wavefront skip the per-element test.
//
// Reference semantics: fusor-ml/fusor/src/composite/flash_attention.rs:141-199, f32 accumulation
// of 16-bit inputs as fusor-ml/core/src/composite/flash_attention.rs:186-203,323-327; head
// mapping kv_head = head / (H / Hkv) (core :135-137,163-167).
#include <type_traits>

#include "attn_bounds.h"
#include "common.h"
#include "device_utils.h"

namespace fhip {

constexpr int PF_WAVES = 8;
constexpr int PF_BM = 32 * PF_WAVES;  // query rows per workgroup
constexpr int PF_BN = 64;             // key rows per tile
constexpr float PF_LOG2E = 1.4426950408889634f;

#define LDS_PTR(type, byte_off) ((__attribute__((address_space(3))) type *)(lds_base + (byte_off)))

template <typename T>
struct Mma;
template <>
struct Mma<half_t> {
    typedef half8_t vec8;
    static __device__ __forceinline__ float16_t mfma(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float x, float y) {
        half2_t h = {(half_t)x, (half_t)y};
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ vec8 scaled(vec8 q, float c) {
#pragma unroll
        for (int e = 0; e < 8; e++) q[e] = (half_t)((float)q[e] * c);
        return q;
    }
};
template <>
struct Mma<bf16_t> {
    typedef bf16x8_t vec8;
    static __device__ __forceinline__ float16_t mfma(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float x, float y) {
        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
        const bf16x2_t h = {(__bf16)x, (__bf16)y};  // v_cvt_pk_bf16_f32: round to nearest even
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ vec8 scaled(vec8 q, float c) {
#pragma unroll
        for (int e = 0; e < 8; e++) q[e] = (__bf16)((float)q[e] * c);
        return q;
    }
};

// LDS image of a 64-row tile.  Rows are kept in 16 groups of 4: row r sits in group r % 16 at
// position r / 16.  A group is exactly what one wavefront-wide direct-to-LDS load writes (4 rows of
// head_dim 16-bit values, contiguous), and groups are padded apart so that
//   - the 16 rows a quarter-wavefront reads for the S^T operand (rows r .. r+15, same 16-byte
//     column) fall 16 bytes apart modulo the 256-byte bank period            (K: pitch 8 D + 16)
//   - the 4 rows x 64 bytes a half-wavefront reads with the transposing load fall 64 bytes apart
//                                                                            (V: pitch 8 D + 64)
template <int D, bool KS>
struct PfCfg {
    static constexpr int ROWB = D * 2;                               // bytes per tile row
    static constexpr int KG = 4 * ROWB + 16;                         // K group pitch, bytes
    static constexpr int VG = 4 * ROWB + 64;                         // V group pitch, bytes
    static constexpr int K_BYTES = 16 * KG;
    static constexpr int V_BYTES = 16 * VG;
    static constexpr int CPR = D / 8;                                // 16-byte chunks per row
    static constexpr int LOAD_LANES = 4 * CPR;                       // lanes of a wavefront-wide tile load (<= 64)
    // tile buffers.  Unsplit form: three stages of (K tile, V tile), tile t in stage t % 3.  Key-split form
    // (KS): a ring of five K tiles followed by a ring of four V tiles (see the slot schedule in the kernel).
    static constexpr int STAGE = K_BYTES + V_BYTES;
    static constexpr int NK = KS ? 5 : 3, NV = KS ? 4 : 3;
    static constexpr int LDS_BYTES = KS ? NK * K_BYTES + NV * V_BYTES : 3 * STAGE;
    static constexpr int BM = KS ? PF_BM / 2 : PF_BM;                // query rows per workgroup
};

__device__ __forceinline__ float half_swap_max(float x) {
    // max of x with the value held by the lane 32 away
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <typename T, int D, bool KS>
__global__ __launch_bounds__(64 * PF_WAVES, 2) void prefill_mfma_kernel(AttnParams p, int nqb, int out_vec) {
    typedef PfCfg<D, KS> C;
    typedef typename Mma<T>::vec8 vec8;
    constexpr int STAGE = C::STAGE;
    constexpr int BM = C::BM;
    __shared__ __attribute__((aligned(16))) char smem[C::LDS_BYTES];
    auto lds_base = (__attribute__((address_space(3))) char *)smem;

    if (p.iv_bad && *p.iv_bad == p.bad_tag) return;  // the mask is not made of intervals: the general kernel takes the call
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: everything derived from it is uniform
    const int lane = tid & 63;
    const int ln = lane & 31;      // query column / key row owned inside a 32-wide MFMA block
    const int h2 = lane >> 5;      // which half of the contraction slice
    const int group = wave >> 2;   // wavefronts w and w + 4 share a SIMD and run out of phase

    // workgroup -> (query block, batch, head): long query blocks first, and heads laid out so
    // the workgroups that land on one XCD (id % 8) share a KV head whenever H is a multiple of 8
    // Packed form (key-split form only, at most 32 query rows, GQA group a multiple of 4): the workgroup's four row
    // blocks are rows 0..31 of four query heads that share a KV head, so the K and V tiles it moves serve all four
    // and a few new rows on a long cache read the cache once per KV head, not once per query head.
    const int pack = KS ? p.pf_pack : 0;
    const int heads = pack ? p.H / 4 : p.H;  // head units per batch entry
    const int bh_count = p.B * heads;
    const int nks = max(p.pf_nsplit, 1);
    const int ksplit = blockIdx.x % nks;  // which share of the keys (0 when the keys are not split over workgroups)
    const int id = blockIdx.x / nks;
    const int qb = nqb - 1 - id / bh_count;
    int rem = id % bh_count;
    const int b = rem / heads;
    int h = rem % heads;
    if (pack) h = 4 * h + (wave & 3);
    else if ((p.H & 7) == 0) h = (h & 7) * (p.H >> 3) + (h >> 3);
    const int g = h / p.G;
    // Rows of a tile beyond the sequence's own keys (kv_lens below the view's length: a ragged batch in one cache
    // allocation) read as zero (the buffers end there): what such rows hold, NaN included, must not reach the result as 0 x NaN in P . V.
    // (likewise the rows behind the last query's own position when the call says where its rows stand inside a longer
    // cache view: a causal descriptor with q_pos_offset + Sq below the view's length)
    int key_end = p.kv_lens ? min(p.Skv, max(p.kv_lens[b], 1)) : p.Skv;
    if (p.analytic && p.causal) key_end = (int)min((int64_t)key_end, max(p.q_pos_offset + p.Sq, (int64_t)1));

    const int q0 = pack ? 0 : qb * BM;
    const int qw0 = pack ? 0 : q0 + 32 * (KS ? (wave & 3) : wave);  // KS: both groups own the same 128 rows
    const int query = qw0 + ln;
    RowBounds rb = row_bounds(p, b, q0, pack ? 32 : BM, qw0, lane);
    if (nks > 1) {  // few query rows on a long cache: this workgroup takes one share of the keys
        const int c_lo = ksplit * p.pf_chunk, c_hi = c_lo + p.pf_chunk;
        rb.lo_wg = max(rb.lo_wg, c_lo), rb.hi_wg = min(rb.hi_wg, c_hi);
        rb.lo_w = max(rb.lo_w, c_lo), rb.hi_w = min(rb.hi_w, c_hi);
        rb.full_lo_w = max(rb.full_lo_w, c_lo), rb.full_hi_w = min(rb.full_hi_w, c_hi);
        rb.klo = max(rb.klo, c_lo), rb.khi = min(rb.khi, c_hi);
    }
    const int lo_wg = rb.lo_wg, hi_wg = rb.hi_wg, lo_w = rb.lo_w, hi_w = rb.hi_w;
    const int full_lo_w = rb.full_lo_w, full_hi_w = rb.full_hi_w, klo = rb.klo, khi = rb.khi;
    const int qrow = min(query, p.Sq - 1);
    const bool wave_has_rows = qw0 < p.Sq;

    // Q^T operand: Q[query][16 kb + 8 h2 .. +8], kept in registers for the whole kernel
    // (the loads are issued here, the scaling waits until the first K/V tiles are on their way too)
    const float scale2 = p.scale * PF_LOG2E;
    // scale2 = pw * rr with pw a power of two and rr in [1, 2).  Q takes pw, which is exact in f16 and bf16 alike, and
    // rr multiplies every score in f32 right before exp2: the scores are then the f32 dot product times the scale, one
    // rounding, as the reference computes them (fusor-ml/fusor/src/composite/flash_attention.rs:145).  Folding all of
    // scale2 into Q instead would save that multiply but round Q's elements a second time (11 bits in f16, 8 in bf16),
    // an error that grows in proportion to the scores.  The S^T accumulators and m are in units of 1 / rr.
    const float pw = __uint_as_float(__float_as_uint(scale2) & 0x7F800000u);
    const float rr = scale2 / pw;
    vec8 qreg[D / 16];
    {
        const uint16_t *qp = (const uint16_t *)p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)qrow * p.qs[2];
#pragma unroll
        for (int kb = 0; kb < D / 16; kb++)
            qreg[kb] = __builtin_bit_cast(vec8, *(const uint4_t *)(qp + 16 * kb + 8 * h2));
    }

    const int j_begin = (lo_wg / PF_BN) * PF_BN;
    const int ntiles = hi_wg > j_begin ? (hi_wg - j_begin + PF_BN - 1) / PF_BN : 0;

    // K and V of this (batch, kv head) as raw buffers: a row beyond the end of the key axis reads as
    // zero, so the tile loop needs neither clamps nor 64-bit address arithmetic
    const uint16_t *kg = (const uint16_t *)p.k + b * p.ks[0] + g * p.ks[1];
    const uint16_t *vg = (const uint16_t *)p.v + b * p.vs[0] + g * p.vs[1];
    const int krow_bytes = (int)p.ks[2] * 2, vrow_bytes = (int)p.vs[2] * 2;

    float16_t o[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.0f;
    // m: the row's reference exponent, in units of the S^T accumulators (1 / rr of a base-2 exponent): probabilities are
    // exp2((s - m) * rr), formed as exp2(fma(s, rr, nmr)) with nmr = -m * rr.  While the row has seen no key m is -inf and
    // nmr +inf, which sends the first tile with a visible key through the branch that sets m (see softmax below).
    float m = -INFINITY, l = 0.0f, nmr = INFINITY;
    float16_t zero16;
#pragma unroll
    for (int r = 0; r < 16; r++) zero16[r] = 0.0f;

    using std::integral_constant;
    // ---- tile movement: global -> LDS directly (no registers) --------------------------------------
    // The four wavefronts of a group move one whole tile with four loads each.  Load j of wavefront w
    // writes LDS group w + 4 j; lane i of it fetches row 16 (i / CPR) + w + 4 j, 16-byte column i % CPR, so
    // the lanes of one load land contiguously (which is what the hardware does with a direct load) and the
    // four loads of a wavefront differ by a uniform offset only.
    // Unsplit form: group 1 moves the K tiles, group 0 the V tiles.  Key-split form: the group that is in
    // its vector phase moves one K and one V tile.
    // The tensors as raw buffer descriptors (base, no stride, size in bytes, 32-bit raw format): a row beyond
    // the end of the key axis reads as zero.
    const bool moves_k = group == 1;
    const int wv = wave & 3;
    auto descriptor = [&](const uint16_t *base, int row_bytes) __attribute__((always_inline)) {
        const uint64_t ptr = (uint64_t)base;
        return uint4_t{(uint32_t)ptr, (uint32_t)(ptr >> 32) & 0xffffu, (uint32_t)((key_end - 1) * row_bytes + D * 2),
                       0x00020000u};
    };
    const uint4_t krs = descriptor(kg, krow_bytes), vrs = descriptor(vg, vrow_bytes);
    const int gofs_k = (16 * (lane / C::CPR) + wv) * krow_bytes + (lane % C::CPR) * 16;
    const int gofs_v = (16 * (lane / C::CPR) + wv) * vrow_bytes + (lane % C::CPR) * 16;
    // where tile t lives in LDS
    auto k_stage = [&](int t) __attribute__((always_inline)) { return KS ? (t % C::NK) * C::K_BYTES : (t % 3) * STAGE; };
    auto v_stage = [&](int t) __attribute__((always_inline)) {
        return KS ? C::NK * C::K_BYTES + (t % C::NV) * C::V_BYTES : (t % 3) * STAGE + C::K_BYTES;
    };
    // a tile that starts beyond the key axis is never used: clamp the (uniform) offset so it stays
    // inside 32 bits; rows past Skv inside a used tile are out of range of the buffer and read 0
    auto issue_loads = [&](const uint4_t rs, int gofs, int row_bytes, int tile, int lbase, int lstep)
                           __attribute__((always_inline)) {
        // (uniform values; pinned to scalar registers, which is what the instruction takes)
        const int soff = __builtin_amdgcn_readfirstlane(min(j_begin + tile * PF_BN, p.Skv) * row_bytes);
        // M0 takes an LDS address, not an offset into the tile buffers (they are the kernel's only LDS variable and
        // start at 0, which the compiler folds in)
        lbase = __builtin_amdgcn_readfirstlane(lbase + (int)(uint32_t)(uintptr_t)lds_base);
        if (C::LOAD_LANES == 64 || lane < C::LOAD_LANES) {
            // written as assembly on purpose: the compiler would otherwise make every later LDS read
            // of this wavefront wait for these loads, whose data is not due before the next barrier
#pragma unroll
            for (int j = 0; j < 4; j++)
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                             :
                             : "s"(lbase + j * lstep), "v"(gofs), "s"(rs), "s"(soff + 4 * j * row_bytes)
                             : "memory", "m0");
        }
    };
    auto issue_k = [&](int tile) __attribute__((always_inline)) {
        issue_loads(krs, gofs_k, krow_bytes, tile, k_stage(tile) + wv * C::KG, 4 * C::KG);
    };
    auto issue_v = [&](int tile) __attribute__((always_inline)) {
        issue_loads(vrs, gofs_v, vrow_bytes, tile, v_stage(tile) + wv * C::VG, 4 * C::VG);
    };
    // unsplit form: this group's tensor, tile `tile`
    const uint4_t mrs = moves_k ? krs : vrs;
    const int mgofs = moves_k ? gofs_k : gofs_v, mrow_bytes = moves_k ? krow_bytes : vrow_bytes;
    const int lds_move_base = (moves_k ? 0 : C::K_BYTES) + wv * (moves_k ? C::KG : C::VG);
    const int lds_move_step = 4 * (moves_k ? C::KG : C::VG);
    auto issue_tile = [&](int tile) __attribute__((always_inline)) {
        issue_loads(mrs, mgofs, mrow_bytes, tile, (tile % 3) * STAGE + lds_move_base, lds_move_step);
    };
    // key-split form, slot s: K(s + 4) and V(s + 1)
    auto issue_slot = [&](int slot) __attribute__((always_inline)) {
        issue_k(slot + 4);
        issue_v(slot + 1);
    };
    // all but the loads of this wavefront's most recent `newer` vector phases have landed
    auto wait_tiles = [&](auto newer) __attribute__((always_inline)) {
        if constexpr (decltype(newer)::value == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        else if constexpr (KS) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    };
    // local tile index -> tile: in the key-split form group g owns the tiles t with t % 2 == g
    auto tile_of = [&](int i) __attribute__((always_inline)) { return KS ? 2 * i + group : i; };

    float16_t s[2];     // S^T of the tile in flight
    uint32_t pk[2][8];  // its probabilities, packed pairs in the MFMA operand order

    // S^T = K . Q^T for this group's tile i (local index; see tile_of)
    auto qk = [&](int i) __attribute__((always_inline)) {
        const int kbase = k_stage(tile_of(i)) + (ln & 15) * C::KG + (ln >> 4) * C::ROWB + h2 * 16;
#pragma unroll
        for (int kb = 0; kb < D / 16; kb++) {
#pragma unroll
            for (int t = 0; t < 2; t++) {
                uint4_t raw = *LDS_PTR(uint4_t, kbase + t * 2 * C::ROWB + kb * 32);
                s[t] = Mma<T>::mfma(__builtin_bit_cast(vec8, raw), qreg[kb], kb == 0 ? zero16 : s[t]);
            }
        }
    };
    // O^T += V^T . P^T for tile i: contraction slice (t, kk) holds this half-wave's keys
    // 32 t + 16 kk + 4 h2 + {0..3} and + 8
    auto pv = [&](int i) __attribute__((always_inline)) {
        const int i16 = lane & 15;
        const int bl = (lane & 31) >> 4;
        const int vbase = v_stage(tile_of(i)) + (4 * h2 + (i16 >> 2)) * C::VG + (16 * bl + 4 * (i16 & 3)) * 2;
#pragma unroll
        for (int gq = 0; gq < 4; gq++) {  // gq = 2 t + kk: rows 16 gq + 4 h2 + {0..3} and + 8
            const int t = gq >> 1, kk = gq & 1;
            const uint4_t braw = {pk[t][4 * kk], pk[t][4 * kk + 1], pk[t][4 * kk + 2], pk[t][4 * kk + 3]};
            const vec8 bop = __builtin_bit_cast(vec8, braw);
#pragma unroll
            for (int db = 0; db < D / 32; db++) {
                const int addr = vbase + gq * C::ROWB + db * 64;
                short4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, addr));
                short4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, addr + 8 * C::VG));
                const uint2_t u0 = __builtin_bit_cast(uint2_t, a0), u1 = __builtin_bit_cast(uint2_t, a1);
                uint4_t araw = {u0[0], u0[1], u1[0], u1[1]};
                o[db] = Mma<T>::mfma(__builtin_bit_cast(vec8, araw), bop, o[db]);
            }
        }
    };
    // Matrix phase in one basic block: S^T of tile ik, then P.V of tile ip.  The first four K operand
    // slices are already in `ka` (read before the barrier that opens the phase, see prefetch_k), so the
    // matrix pipe starts at once; the remaining LDS reads are issued several MFMAs ahead of their use
    // (the order is pinned by the scheduling groups at the end; without them the reads sit right in
    // front of their MFMAs and the pipe waits out the LDS latency every few instructions).
    constexpr int PFK = (D == 128) ? 2 : 4;  // K operand slices in flight (register budget)
    uint4_t ka[PFK][2];
    auto prefetch_k = [&](int ik) __attribute__((always_inline)) {
        const int kbase = k_stage(tile_of(ik)) + (ln & 15) * C::KG + (ln >> 4) * C::ROWB + h2 * 16;
#pragma unroll
        for (int kb = 0; kb < PFK; kb++)
#pragma unroll
            for (int t = 0; t < 2; t++) ka[kb][t] = *LDS_PTR(uint4_t, kbase + t * 2 * C::ROWB + kb * 32);
    };
    auto qk_pv = [&](int ip, int ik, auto do_pv, auto prefetched) __attribute__((always_inline)) {
        constexpr bool PV = decltype(do_pv)::value;
        constexpr bool PRE = decltype(prefetched)::value;
        constexpr int NDB = D / 32, NKB = D / 16;
        const int vstage = v_stage(tile_of(ip)), kstage = k_stage(tile_of(ik));
        const int i16 = lane & 15;
        const int bl = (lane & 31) >> 4;
        const int vbase = vstage + (4 * h2 + (i16 >> 2)) * C::VG + (16 * bl + 4 * (i16 & 3)) * 2;
        const int kbase = kstage + (ln & 15) * C::KG + (ln >> 4) * C::ROWB + h2 * 16;
        uint4_t va[2][NDB];
        auto read_v = [&](int gq, uint4_t (&a)[NDB]) {  // gq = 2 t + kk: rows 32 t + 16 kk (+8)
#pragma unroll
            for (int db = 0; db < NDB; db++) {
                const int addr = vbase + gq * C::ROWB + db * 64;
                short4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, addr));
                short4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, addr + 8 * C::VG));
                const uint2_t u0 = __builtin_bit_cast(uint2_t, a0), u1 = __builtin_bit_cast(uint2_t, a1);
                a[db] = uint4_t{u0[0], u0[1], u1[0], u1[1]};
            }
        };
        auto mfma_v = [&](int gq, const uint4_t (&a)[NDB]) {
            const int t = gq >> 1, kk = gq & 1;
            const uint4_t braw = {pk[t][4 * kk], pk[t][4 * kk + 1], pk[t][4 * kk + 2], pk[t][4 * kk + 3]};
            const vec8 bop = __builtin_bit_cast(vec8, braw);
#pragma unroll
            for (int db = 0; db < NDB; db++) o[db] = Mma<T>::mfma(__builtin_bit_cast(vec8, a[db]), bop, o[db]);
        };
        auto read_k = [&](int kb, uint4_t (&a)[2]) {
#pragma unroll
            for (int t = 0; t < 2; t++) a[t] = *LDS_PTR(uint4_t, kbase + t * 2 * C::ROWB + kb * 32);
        };
        if constexpr (!PRE) {
#pragma unroll
            for (int kb = 0; kb < PFK; kb++) read_k(kb, ka[kb]);
        }
#pragma unroll
        for (int kb = 0; kb < NKB; kb++) {
#pragma unroll
            for (int t = 0; t < 2; t++)
                s[t] = Mma<T>::mfma(__builtin_bit_cast(vec8, ka[kb % PFK][t]), qreg[kb], kb == 0 ? zero16 : s[t]);
            if (kb + PFK < NKB) read_k(kb + PFK, ka[kb % PFK]);
            if (PV && kb >= NKB - 4 && kb < NKB - 2) read_v(kb + 4 - NKB, va[kb + 4 - NKB]);
        }
        if constexpr (PV) {
            mfma_v(0, va[0]);
            read_v(2, va[0]);
            mfma_v(1, va[1]);
            read_v(3, va[1]);
            mfma_v(2, va[0]);
            mfma_v(3, va[1]);
        }
        // scheduling groups: 0x100 = LDS read, 0x008 = MFMA
        auto constexpr_reads = [&](int kb) __attribute__((always_inline)) {
            const bool rk = kb + PFK < NKB, rv = PV && kb >= NKB - 4 && kb < NKB - 2;
            if (rk && rv) __builtin_amdgcn_sched_group_barrier(0x100, 2 + 2 * NDB, 0);
            else if (rk) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            else if (rv) __builtin_amdgcn_sched_group_barrier(0x100, 2 * NDB, 0);
        };
        if constexpr (!PRE) __builtin_amdgcn_sched_group_barrier(0x100, 2 * PFK, 0);
#pragma unroll
        for (int kb = 0; kb < NKB; kb++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            constexpr_reads(kb);
        }
        if constexpr (PV) {
            __builtin_amdgcn_sched_group_barrier(0x008, NDB, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * NDB, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, NDB, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * NDB, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 2 * NDB, 0);
        }
    };
    // mask + online softmax (log2 domain, lazily rescaled) of tile i: s -> pk
    auto softmax = [&](int i) __attribute__((always_inline)) {
        const int j0 = j_begin + tile_of(i) * PF_BN;
        if (!(j0 >= full_lo_w && j0 + PF_BN <= full_hi_w)) {
            // element r of block t is key j0 + 32 t + 8 (r / 4) + 4 h2 + r % 4
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int key = j0 + 32 * t + 8 * (r >> 2) + 4 * h2 + (r & 3);
                    s[t][r] = (key >= klo && key < khi) ? s[t][r] : -INFINITY;
                }
        }
        // Probabilities against the reference the row already has; no maximum is taken.  The reference is whatever maximum
        // the row had when it was last set, so a probability may exceed 1: harmless while it stays inside the 16-bit
        // type's range (P is rounded to it for the second product; l and O are f32), and that is what the check below
        // guarantees: a lane's 32 probabilities are positive, so while their sum is at most 2^15 each of them is.
        auto probabilities = [&](float nm) __attribute__((always_inline)) {
            float ts = 0.0f;
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][r], rr, nm));
                    const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][r + 1], rr, nm));
                    pk[t][r >> 1] = Mma<T>::pack2(p0, p1);
                    ts += p0 + p1;  // plain f32 adds: a dot-product instruction here would queue behind the MFMAs
                }
            return ts;
        };
        float ts = probabilities(nmr);
        // Not at most 2^15 (which also catches the +inf and NaN a row without a reference produces): some row of the
        // wavefront needs its reference moved.  Take the tile's maximum, move every row's reference to at least that,
        // rescale what the row has accumulated, and form the tile's probabilities again.
        if (__builtin_amdgcn_ballot_w64(!(ts <= 32768.0f)) != 0) {
            float mx = s[0][0];
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[t][r]);
            mx = half_swap_max(mx);
            const float m_new = fmaxf(m, mx);
            const float corr = (m == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f((m - m_new) * rr);
            m = m_new;
            l *= corr;
#pragma unroll
            for (int db = 0; db < D / 32; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[db][r] *= corr;
            // still no visible key: the tile's probabilities are exp2(-inf) = 0 and the row stays without a reference
            nmr = (m == -INFINITY) ? INFINITY : -m * rr;
            ts = probabilities((m == -INFINITY) ? 0.0f : nmr);
        }
        l += ts;
    };

    // ---- slot schedule ---------------------------------------------------------------------------------
    // Slots are separated by workgroup barriers.  Group 0 is in its matrix phase in even slots and in
    // its vector phase in odd slots; group 1 the other way round, one slot later.  Matrix phase of
    // tile i: S^T of tile i (reads K(i)), then P.V of tile i-1 (reads V(i-1)); K(i) is read in slots 2i
    // and 2i+1, V(i) in slots 2i+2 and 2i+3.  Vector phase: issue a tile load, softmax, read the first
    // K operands of the next matrix phase, wait for the tile load issued one vector phase earlier.
    // Tile t lives in stage t % 3.  In even slot 2j group 1 issues K(j+2) (its stage was last read for
    // K(j-1) in slot 2j-1) and makes sure K(j+1) has landed; in odd slot 2j+1 group 0 issues V(j+1)
    // (stage last read for V(j-2) in slot 2j-1) and makes sure V(j) has landed.  Every tile is thus
    // complete, and published by a barrier, before the slot of its first reader, and has had two
    // slots to arrive.
    // The tiles visible to a wavefront form one contiguous range [ia, ib).  Each group walks the slot
    // sequence in five static segments (nothing / first tile / steady state / last tile / nothing) so
    // that the steady-state loop body is branch-free and no state changes registers between phases.
    //
    // Key-split form (KS): both groups own the same 128 rows and group g takes the tiles t with t % 2 == g,
    // so a slot is the matrix phase of tile s for one group and the vector phase of tile s-1 for the other;
    // the groups' (m, l, O) are merged at the end.  K(t) is read in slot t (its first operands at the end of
    // slot t-1), V(t) in slot t+2.  The group in its vector phase in slot s issues K(s+4) into the stage K(s-1)
    // has just left (ring of 5) and V(s+1) into the stage of V(s-3), last read in slot s-1 (ring of 4), and
    // makes sure its loads of slot s-2, K(s+2) and V(s-1), have landed: each is published by a barrier one
    // slot before its first reader and has had two slots to arrive.  The segments below then run on the
    // group's own tile count: local tile i of group g is tile 2 i + g.
    int ia = 0, ib = 0;
    if (wave_has_rows && hi_w > lo_w) {
        ia = (lo_w - j_begin) / PF_BN;
        ib = min(ntiles, (hi_w - j_begin + PF_BN - 1) / PF_BN);
        if (ib < ia) ib = ia;
    }
    int n_iter = ntiles + 1;  // iterations (two slots each) of either group
    if constexpr (KS) {
        ia = (ia + 1 - group) >> 1;  // this group's tiles below ia / below ib
        ib = (ib + 1 - group) >> 1;
        n_iter = (ntiles + 3) >> 1;
    }
    // MODE bit 0: S^T of tile i; bit 1: P.V of tile i-1; bit 2: softmax of tile i (group 0) / i-1 (group 1);
    // bit 3: the K operands of tile i were prefetched by the preceding vector phase
    auto matrix_phase = [&](int i, auto mode) __attribute__((always_inline)) {
        constexpr int MODE = decltype(mode)::value;
        __builtin_amdgcn_s_setprio(1);
        if constexpr ((MODE & 11) == 11) qk_pv(i - 1, i, std::true_type{}, std::true_type{});
        else if constexpr ((MODE & 11) == 9) qk_pv(i - 1, i, std::false_type{}, std::true_type{});
        else {
            if constexpr ((MODE & 2) != 0) pv(i - 1);
            if constexpr ((MODE & 1) != 0) qk(i);
        }
        __builtin_amdgcn_s_setprio(0);
    };
    // next_k: the tile whose S^T this wavefront computes in its next matrix phase
    auto vector_phase = [&](int i, int tile_to_load, int slot, int next_k, auto mode) __attribute__((always_inline)) {
        constexpr int MODE = decltype(mode)::value;
        if constexpr (KS) issue_slot(slot);
        else issue_tile(tile_to_load);
        if constexpr ((MODE & 4) != 0) softmax(i);
        if constexpr ((MODE & 16) != 0) prefetch_k(next_k);
        wait_tiles(integral_constant<int, 1>{});  // the tile issued one vector phase ago has landed
    };
    // MODE bit 4: prefetch the K operands for the next matrix phase at the end of the vector phase
    auto segment0 = [&](int i0, int i1, auto mode) __attribute__((always_inline)) {  // group 0: slot 2i matrix, slot 2i+1 vector + V(i)
        for (int i = i0; i < i1; i++) {
            matrix_phase(i, mode);
            lds_barrier();
            vector_phase(i, i + 1, 2 * i + 1, i + 1, mode);
            lds_barrier();
        }
    };
    auto segment1 = [&](int i0, int i1, auto mode) __attribute__((always_inline)) {  // group 1: slot 2i vector (tile i-1) + K(i+1), slot 2i+1 matrix
        for (int i = i0; i < i1; i++) {
            vector_phase(i - 1, i + 2, 2 * i, i, mode);
            lds_barrier();
            matrix_phase(i, mode);
            lds_barrier();
        }
    };
    if (ntiles > 0) {
        if constexpr (KS) {  // what slots -4 .. -1 would have issued
            if (group == 0) {
                issue_k(0);
                issue_k(2);
                issue_v(0);
            } else {
                issue_k(1);
                issue_k(3);
            }
        } else if (moves_k) {
            issue_tile(0);
            issue_tile(1);
        } else {
            issue_tile(0);
        }
#pragma unroll
        for (int kb = 0; kb < D / 16; kb++) qreg[kb] = Mma<T>::scaled(qreg[kb], pw);
        wait_tiles(integral_constant<int, 0>{});
        lds_barrier();
        if (group == 0) {
            // iteration i: S^T(i), softmax(i), P.V(i-1)
            segment0(0, ia, integral_constant<int, 0>{});
            if (ia < ib) {
                segment0(ia, ia + 1, integral_constant<int, 1 | 4 | 16>{});
                segment0(ia + 1, ib, integral_constant<int, 1 | 2 | 4 | 8 | 16>{});
                segment0(ib, ib + 1, integral_constant<int, 2>{});
                segment0(ib + 1, n_iter, integral_constant<int, 0>{});
            } else {
                segment0(ia, n_iter, integral_constant<int, 0>{});
            }
        } else {
            // iteration i: softmax(i-1), then S^T(i) and P.V(i-1)
            segment1(0, ia, integral_constant<int, 0>{});
            if (ia < ib) {
                segment1(ia, ia + 1, integral_constant<int, 1 | 8 | 16>{});
                segment1(ia + 1, ib, integral_constant<int, 1 | 2 | 4 | 8 | 16>{});
                segment1(ib, ib + 1, integral_constant<int, 2 | 4>{});
                segment1(ib + 1, n_iter, integral_constant<int, 0>{});
            } else {
                segment1(ia, n_iter, integral_constant<int, 0>{});
            }
        }
    }

    // the epilogue reuses the tile buffers: no tile load may still be on its way into them
    wait_tiles(integral_constant<int, 0>{});
    lds_barrier();
    constexpr int SLICE = 32 * (D * 2 + 16);  // bytes per wavefront of the output transposition below
    if constexpr (KS) {
        // Group 1 hands its state to group 0, which holds the other half of the keys of the same rows:
        // log-sum-exp merge, as the split-KV combine does.  One f32 per lane per slot, above the slices the
        // output transposition uses.
        constexpr int PARK = 4 * SLICE;
        constexpr int NSLOT = D / 2 + 2;
        static_assert(PARK + NSLOT * 1024 <= C::LDS_BYTES, "merge area exceeds the tile buffers");
        auto park = (__attribute__((address_space(3))) float *)(lds_base + PARK) + (wave & 3) * 64 + lane;
        if (group == 1) {
#pragma unroll
            for (int db = 0; db < D / 32; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) park[(db * 16 + r) * 256] = o[db][r];
            park[(D / 2) * 256] = m;
            park[(D / 2 + 1) * 256] = l;
        }
        lds_barrier();
        if (group == 1) return;
        const float m1 = park[(D / 2) * 256], l1 = park[(D / 2 + 1) * 256];
        const float mn = fmaxf(m, m1);
        const float c0 = (m == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f((m - mn) * rr);
        const float c1 = (m1 == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f((m1 - mn) * rr);
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[db][r] = o[db][r] * c0 + park[(db * 16 + r) * 256] * c1;
        l = l * c0 + l1 * c1;
        m = mn;
    }
    // ---- epilogue: out[query][dim] = O^T[dim][query] / l ----------------------------------------------
    const float l_tot = half_swap_sum(l);
    // With the keys split over workgroups the "output" is this share's row in the partials: O unnormalised
    // as f32 in 16-byte pieces, then (m, l); the merge kernel normalises.
    const bool parked = nks > 1;
    const float inv = parked ? 1.0f : 1.0f / l_tot;
    const bool dead = !parked && (l_tot == 0.0f);  // no visible key: the reference gives NaN (0/0)
    const bool out_f32 = parked || p.out_f32;
    const int64_t os0 = parked ? (int64_t)p.H * p.Sq * nks * p.pf_pitch : p.os[0];
    const int64_t os1 = parked ? (int64_t)p.Sq * nks * p.pf_pitch : p.os[1];
    const int64_t os2 = parked ? (int64_t)nks * p.pf_pitch : p.os[2];
    char *const og = parked ? (char *)(p.partials + (int64_t)ksplit * p.pf_pitch) : (char *)p.out;
    if (parked && query < p.Sq && h2 == 0) {
        float *ws = (float *)og + b * os0 + h * os1 + (int64_t)query * os2;
        ws[D] = m * rr;  // base-2 exponent units
        ws[D + 1] = l_tot;
    }
    if (out_vec || parked) {
        // transpose through a wavefront-private slice of the LDS so that every global store is a
        // 16-byte piece of a contiguous row; 32 rows per round for 2-byte outputs, 16 for f32
        const int esz = out_f32 ? 4 : 2;
        const int pitch = D * esz + 16;                      // rows stay 16-byte aligned, 4 banks apart
        static_assert(PF_WAVES * SLICE <= C::LDS_BYTES, "epilogue staging exceeds the tile buffers");
        auto wbase = lds_base + wave * SLICE;
        const int rounds = out_f32 ? 2 : 1;
        const int rows_per_round = 32 / rounds;
        const int cpr = D * esz / 16;
        for (int rd = 0; rd < rounds; rd++) {
            const int row_lo_ = rd * rows_per_round;
            if (ln >= row_lo_ && ln < row_lo_ + rows_per_round) {
#pragma unroll
                for (int db = 0; db < D / 32; db++)
#pragma unroll
                    for (int rq = 0; rq < 4; rq++) {
                        float v4[4];
#pragma unroll
                        for (int e = 0; e < 4; e++) v4[e] = dead ? __builtin_nanf("") : o[db][4 * rq + e] * inv;
                        const int dim = 32 * db + 8 * rq + 4 * h2;
                        if (out_f32) {
                            *(__attribute__((address_space(3))) float4_t *)(wbase + (ln - row_lo_) * pitch + dim * 4) =
                                float4_t{v4[0], v4[1], v4[2], v4[3]};
                        } else {
                            const uint2_t pk2 = {Mma<T>::pack2(v4[0], v4[1]), Mma<T>::pack2(v4[2], v4[3])};
                            *(__attribute__((address_space(3))) uint2_t *)(wbase + ln * pitch + dim * 2) = pk2;
                        }
                    }
            }
            wave_lds_sync();
            for (int c = lane; c < rows_per_round * cpr; c += 64) {
                const int row = c / cpr, col = c % cpr;
                const int qr = qw0 + row_lo_ + row;
                if (qr < p.Sq) {
                    const uint4_t val = *(__attribute__((address_space(3))) uint4_t *)(wbase + row * pitch + col * 16);
                    const int64_t eidx = b * os0 + h * os1 + (int64_t)qr * os2;
                    *(uint4_t *)(og + eidx * esz + col * 16) = val;
                }
            }
            wave_lds_sync();
        }
    } else if (query < p.Sq) {
        const int64_t obase = b * p.os[0] + h * p.os[1] + (int64_t)query * p.os[2];
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int dim = 32 * db + 8 * (r >> 2) + 4 * h2 + (r & 3);
                const float val = dead ? __builtin_nanf("") : o[db][r] * inv;
                if (p.out_f32) ((float *)p.out)[obase + dim * p.os[3]] = val;
                else ((T *)p.out)[obase + dim * p.os[3]] = from_float<T>(val);
            }
    }
}

// Query blocks of 256 rows leave CUs idle when there are few of them (short prompts, a few new rows on a long
// cache), and a causal prompt's last blocks are several times longer than its first.  The key-split form (128
// rows, twice the workgroups, the longest one half as long) costs about 7 % per tile and a longer prologue and
// epilogue; measured, it wins (1.1-1.35 x) while the 256-row grid fills at most half the CUs, for up to 128
// query rows (where the second wavefront group would have no rows at all), and for one workgroup per CU when a
// head has 8 or more query blocks; it loses with fewer than three key tiles.
static bool use_key_split_form(const AttnParams &p) {
    const int cus = p.cus > 0 ? p.cus : 256;
    const int nqb = (p.Sq + PF_BM - 1) / PF_BM;
    const long wgs = (long)nqb * p.B * p.H * (p.pf_nsplit > 1 ? p.pf_nsplit : 1);
    if (p.Skv <= 2 * PF_BN) return false;
    return p.Sq <= PF_BM / 2 || 2 * wgs <= cus || (wgs <= cus && nqb >= 8);
}

template <typename T>
static int launch_t(const AttnParams &p0, hipStream_t stream) {
    AttnParams p = p0;
    const bool ks = use_key_split_form(p);
    p.pf_pack = ks ? prefill_mfma_pack(p.B, p.H, p.G, p.Sq, p.Skv, p.cus > 0 ? p.cus : 256) : 0;
    const int bm = ks ? PF_BM / 2 : PF_BM;
    const int nqb = p.pf_pack ? 1 : (p.Sq + bm - 1) / bm;
    const long blocks = (long)nqb * p.B * (p.pf_pack ? p.H / 4 : p.H) * (p.pf_nsplit > 1 ? p.pf_nsplit : 1);
    if (blocks > 0x7fffffffL) {
        set_error("prefill: too many workgroups (%ld)", blocks);
        return FHIP_ERR_UNSUPPORTED;
    }
    dim3 grid((unsigned)blocks), block(64 * PF_WAVES);
    // rows of the output can be written in 16-byte pieces when they are contiguous and aligned
    const int oeb = p.out_f32 ? 4 : 2;
    int out_vec = (p.os[3] == 1 || p.D == 1) && ((uintptr_t)p.out % 16 == 0);
    for (int i = 0; i < 3; i++)
        if ((p.os[i] * oeb) % 16 != 0) out_vec = 0;
#define PF_LAUNCH(DIM)                                                                                         \
    if (ks) FHIP_LAUNCH_MAIN((prefill_mfma_kernel<T, DIM, true>), grid, block, stream, p, p, nqb, out_vec);      \
    else FHIP_LAUNCH_MAIN((prefill_mfma_kernel<T, DIM, false>), grid, block, stream, p, p, nqb, out_vec)
    switch (p.D) {
        case 64: PF_LAUNCH(64); break;
        case 96: PF_LAUNCH(96); break;
        case 128: PF_LAUNCH(128); break;
        default: set_error("prefill MFMA kernel: head_dim %d not in {64, 96, 128}", p.D); return FHIP_ERR_UNSUPPORTED;
    }
#undef PF_LAUNCH
    FHIP_HIP_CHECK(hipGetLastError());
    if (p.pf_nsplit > 1) return launch_prefill_merge(p, sizeof(T) == 2 && std::is_same<T, half_t>::value ? FHIP_F16 : FHIP_BF16, stream);
    return FHIP_OK;
}

// Few query rows on a long cache: 256-row query blocks alone leave most CUs idle, so the keys are split over
// workgroups too, down to 1024 keys per share, until there are about two workgroups per CU.
// Query heads per workgroup of the packed form (0: not packed).  Packing divides the workgroups by four, and a share of
// the keys is at least 1024 keys long, so it is taken when the packed grid still reaches half the CUs (12..32 rows:
// batch 8 on 8192 keys 98 -> 66..81 us, batch 4 on 4096 keys 45 -> 28 us, batch 1 on 32768 keys 68 -> 40 us; with a
// quarter of the CUs, batch 1 on 8192 keys, the unpacked grid is as quick: 25.7 against 26.5 us).
int prefill_mfma_pack(int B, int H, int G, int Sq, int Skv, int compute_units) {
    if (!(Sq <= 32 && G >= 4 && G % 4 == 0) || Skv <= 2 * PF_BN) return 0;
    const long shares = Skv / 1024 > 1 ? Skv / 1024 : 1;
    return 2 * (long)B * (H / 4) * shares >= compute_units ? 4 : 0;
}

void prefill_mfma_plan(int B, int H, int G, int Sq, int Skv, bool causal_square, int compute_units, int *nsplit, int *chunk) {
    *nsplit = 1;
    *chunk = Skv;
    if (causal_square) return;
    const long wgs = (long)B * (prefill_mfma_pack(B, H, G, Sq, Skv, compute_units) ? H / 4 : H) * ((Sq + PF_BM - 1) / PF_BM);
    if (2 * wgs > compute_units) return;  // the query blocks alone keep at least half the chip busy: parking and
                                          // merging partial results would cost more than it gains (measured)
    const long want = (2L * compute_units + wgs - 1) / wgs;
    long most = Skv / 1024;
    // A few rows on a short cache: shares down to 512 keys, and for up to 64 rows to 256, while CUs would stay without a
    // workgroup (f16, 32/8 heads, head_dim 128, B1: 12...32 rows on 2048 keys 24.6 -> 17.8 us, on 4096 keys 24.7 -> 20.7;
    // 128 rows on 2048 keys 28.8 -> 25.7).  On 1024 keys two shares of 512 lose with more than 64 rows (21.2 -> 23.4 us).
    const bool few_rows = 2L * Sq <= Skv && (Sq <= 64 || Skv >= 2048);
    if (few_rows && (want < most ? want : most) * wgs < compute_units) most = Skv / 512;
    if (few_rows && Sq <= 64 && (want < most ? want : most) * wgs < compute_units) most = Skv / 256;
    long ns = want < most ? want : most;
    if (ns < 2) return;
    long c = (Skv + ns - 1) / ns;
    c = (c + PF_BN - 1) / PF_BN * PF_BN;
    *chunk = (int)c;
    *nsplit = (int)((Skv + c - 1) / c);
}

size_t prefill_mfma_workspace_bytes(int B, int H, int Sq, int D, int nsplit) {
    if (nsplit <= 1) return 0;
    return (size_t)B * H * Sq * nsplit * (size_t)(D + 4) * sizeof(float);
}

int launch_prefill_mfma(const AttnParams &p, fhip_dtype dtype, hipStream_t stream) {
    if (dtype == FHIP_F16) return launch_t<half_t>(p, stream);
    if (dtype == FHIP_BF16) return launch_t<bf16_t>(p, stream);
    set_error("prefill MFMA kernel takes f16/bf16 only");
    return FHIP_ERR_UNSUPPORTED;
}

}  // namespace fhip
