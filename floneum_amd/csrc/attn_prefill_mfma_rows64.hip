// Prefill attention for f16 / bf16 at head_dim 128 with 64 query rows per wavefront: four wavefronts per workgroup, one
// per SIMD with the whole register file, 256 query rows per workgroup.
//
// The 256-row kernel of attn_prefill_mfma.hip runs eight wavefronts of 32 rows: every K and V operand a wavefront reads
// from LDS feeds ONE v_mfma_f32_32x32x16, and each of the eight reads the whole tile.  Here a wavefront owns two 32-row
// blocks, Q (64 registers) and O^T (128) of both in registers, and every operand it reads feeds TWO matrix
// instructions: half the LDS instructions and bytes per matrix instruction.  With one wavefront per SIMD nothing
// overlaps unless the instruction stream itself interleaves it, so the loop is software-pipelined over 32-key
// sub-tiles as in attn_prefill_mfma_rows32.hip.  For sub-tile t:
//   block B:  O^T += V(t-1)^T . P(t-1)^T on the matrix pipe; beside it the LDS hands over the rest of V(t-1)'s operands,
//             the first of K(t+1)'s and the first of V(t)'s, the vector ALU turns the first row block's scores S^T(t)
//             into probabilities, and tile loads are issued
//   block A:  S^T(t+1) = K(t+1) . Q^T on the matrix pipe; beside it the vector ALU turns the second row block's scores
//             S^T(t) into probabilities and the LDS hands over the rest of K(t+1)'s operands
// The scores accumulate in vector registers, where the softmax reads them, and scores and probabilities are kept twice,
// by the sub-tile's parity (the matrix pipe writes S^T(t+1) while the vector ALU reads S^T(t), and reads P(t-1) while
// the vector ALU writes P(t)): the loop body is two sub-tiles.
// Each block is sixteen steps of one matrix instruction and what runs beside it, fenced so that the compiler keeps
// them apart.  K and V live in rings of four 64-key LDS tiles each (two sub-tiles per tile, the LDS image of the
// 256-row kernel), loaded straight into LDS: an iteration is two sub-tiles and issues one K tile in its first half and
// one V tile in its second, each a whole iteration and a barrier ahead of its first reader; the one workgroup barrier
// per iteration publishes what has landed.
//
// Softmax as in the 256-row kernel: Q carries the power-of-two part of scale * log2(e), the rest (rr in [1, 2))
// multiplies the scores in f32; a probability is exp2(fma(s, rr, -m * rr)) against the reference m the row already
// has, and m moves only when a lane's probabilities of a tile sum to more than 2^15.
// Masking is by interval (attn_bounds.h): analytic descriptors, key counts, the interval form of a mask tensor; the
// scores of a sub-tile that is not visible to all of the wavefront's rows get their -inf before the softmax reads them.
// Two branches per sub-tile stay on the path of every sub-tile (must a reference move; does the next sub-tile need its
// mask): merged into one, or with the next block's addresses formed ahead of them, the kernel measured slower.
//
// Reference semantics: fusor-ml/fusor/src/composite/flash_attention.rs:141-199 with the f32 accumulation of 16-bit
// inputs of fusor-ml/core/src/composite/flash_attention.rs:186-203,323-327.
#include <type_traits>

#include "attn_bounds.h"
#include "common.h"
#include "device_utils.h"

namespace fhip {

namespace {

constexpr float R64_LOG2E = 1.4426950408889634f;
constexpr int R64_D = 128;     // the kernel's head dim
constexpr int R64_BM = 256;    // query rows per workgroup
constexpr int R64_RB = 2;      // 32-row blocks per wavefront
constexpr int R64_KEYS = 32;   // keys per sub-tile (one loop iteration)
constexpr int R64_TILE = 64;   // keys per LDS tile
// LDS image of a 64-row tile: rows in 16 groups of 4 (row r in group r % 16 at position r / 16), a group being what one
// wavefront-wide direct load writes (1 KB), and groups padded apart so that the 16 rows a quarter-wavefront reads for
// the S^T operand fall 16 bytes apart modulo the 256-byte bank period (K) and the 4 rows x 64 bytes a half-wavefront
// reads with the transposing load fall 64 bytes apart (V).  Sub-tile s of a tile is positions 2 s and 2 s + 1.
constexpr int R64_ROWB = R64_D * 2;
constexpr int R64_KG = 4 * R64_ROWB + 16;
constexpr int R64_VG = 4 * R64_ROWB + 64;
constexpr int R64_K_BYTES = 16 * R64_KG;
constexpr int R64_V_BYTES = 16 * R64_VG;
constexpr int R64_NK = 4, R64_NV = 4;
constexpr int R64_V_AT = R64_NK * R64_K_BYTES;
constexpr int R64_LDS_BYTES = R64_V_AT + R64_NV * R64_V_BYTES;

#define R64_LDS(type, byte_off) ((__attribute__((address_space(3))) type *)(lds_base + (byte_off)))

template <typename T>
struct R64Mma;
template <>
struct R64Mma<half_t> {
    typedef half8_t vec8;
    static __device__ __forceinline__ float16_t mfma(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    // S^T accumulators live in the vector half of the register file, where the softmax reads them: the builtin leaves
    // the choice to the compiler, which keeps every accumulator of a kernel that pins operands to the accumulation half
    // there, and 32 moves per sub-tile follow.  (Nothing reads a score sooner than a block after its last matrix
    // instruction, and the matrix instructions of a chain are two apart: no wait states are owed.)
    static __device__ __forceinline__ void mfma_first_v(float16_t &d, uint4_t a, vec8 b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(d) : "a"(a), "v"(b));
    }
    static __device__ __forceinline__ void mfma_v(float16_t &d, uint4_t a, vec8 b) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "a"(a), "v"(b));
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
struct R64Mma<bf16_t> {
    typedef bf16x8_t vec8;
    static __device__ __forceinline__ float16_t mfma(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void mfma_first_v(float16_t &d, uint4_t a, vec8 b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "a"(a), "v"(b));
    }
    static __device__ __forceinline__ void mfma_v(float16_t &d, uint4_t a, vec8 b) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "a"(a), "v"(b));
    }
    static __device__ __forceinline__ uint32_t pack2(float x, float y) {
        typedef __bf16 bf16x2r_t __attribute__((ext_vector_type(2)));
        const bf16x2r_t h = {(__bf16)x, (__bf16)y};  // v_cvt_pk_bf16_f32: round to nearest even
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ vec8 scaled(vec8 q, float c) {
#pragma unroll
        for (int e = 0; e < 8; e++) q[e] = (__bf16)((float)q[e] * c);
        return q;
    }
};

__device__ __forceinline__ float r64_half_swap_max(float x) {  // max of x with the value held by the lane 32 away
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float r64_half_swap_sum(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <typename T>
__global__ __launch_bounds__(256, 1) void prefill_mfma_rows64_kernel(AttnParams p, int nqb, int out_vec) {
    typedef typename R64Mma<T>::vec8 vec8;
    constexpr int D = R64_D, ROWB = R64_ROWB, KG = R64_KG, VG = R64_VG, RB = R64_RB;
    constexpr int KB = D / 16;  // contraction slices of S^T
    constexpr int DB = D / 32;  // 32-dim blocks of O^T
    __shared__ __attribute__((aligned(16))) char smem[R64_LDS_BYTES];
    auto lds_base = (__attribute__((address_space(3))) char *)smem;

    if (p.iv_bad && *p.iv_bad == p.bad_tag) return;  // the mask is not made of intervals: the kernel behind takes the call
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int ln = lane & 31;  // query column / key row owned inside a 32-wide block
    const int h2 = lane >> 5;  // which half of the contraction slice
    const int hd = p.D;

    // workgroup -> (query block, batch, head): long (late) query blocks first; consecutive workgroups land on
    // consecutive XCDs, so with H a multiple of 8 the heads are dealt so that an XCD works on neighbouring heads
    const int bh_count = p.B * p.H;
    const int id = blockIdx.x;
    const int qb = nqb - 1 - id / bh_count;
    const int rem = id % bh_count;
    const int b = rem / p.H;
    int h = rem % p.H;
    if ((p.H & 7) == 0) h = (h & 7) * (p.H >> 3) + (h >> 3);
    const int g = h / p.G;
    // rows of a tile beyond the sequence's own keys read as zero (the buffers end there)
    int key_end = p.kv_lens ? min(p.Skv, max(p.kv_lens[b], 1)) : p.Skv;
    if (p.analytic && p.causal) key_end = (int)min((int64_t)key_end, max(p.q_pos_offset + p.Sq, (int64_t)1));

    const int q0 = qb * R64_BM, qw0 = q0 + 32 * RB * wave;
    int klo[RB], khi[RB], query[RB], qrow[RB];
    int lo_wg, hi_wg, full_lo_w, full_hi_w, lo_w, hi_w;
    {
        const RowBounds r0 = row_bounds(p, b, q0, R64_BM, qw0, lane);
        const RowBounds r1 = row_bounds(p, b, q0, R64_BM, qw0 + 32, lane);
        klo[0] = r0.klo, khi[0] = r0.khi, klo[1] = r1.klo, khi[1] = r1.khi;
        lo_wg = __builtin_amdgcn_readfirstlane(r0.lo_wg), hi_wg = __builtin_amdgcn_readfirstlane(r0.hi_wg);
        full_lo_w = __builtin_amdgcn_readfirstlane(max(r0.full_lo_w, r1.full_lo_w));
        full_hi_w = __builtin_amdgcn_readfirstlane(min(r0.full_hi_w, r1.full_hi_w));
        // union over the wavefront's 64 rows (a row block without a visible key reports the empty interval [0, 0))
        const bool e0 = r0.hi_w <= r0.lo_w, e1 = r1.hi_w <= r1.lo_w;
        lo_w = __builtin_amdgcn_readfirstlane(e0 ? r1.lo_w : e1 ? r0.lo_w : min(r0.lo_w, r1.lo_w));
        hi_w = __builtin_amdgcn_readfirstlane(e0 ? r1.hi_w : e1 ? r0.hi_w : max(r0.hi_w, r1.hi_w));
    }
#pragma unroll
    for (int rb = 0; rb < RB; rb++) query[rb] = qw0 + 32 * rb + ln, qrow[rb] = min(query[rb], p.Sq - 1);

    const float scale2 = p.scale * R64_LOG2E;
    // scale2 = pw * rr with pw a power of two and rr in [1, 2): Q takes pw (exact), rr multiplies every score in f32
    const float pw = __uint_as_float(__float_as_uint(scale2) & 0x7F800000u);
    const float rr = scale2 / pw;

    const int j_begin = (lo_wg / R64_TILE) * R64_TILE;
    const int ntiles = hi_wg > j_begin ? (hi_wg - j_begin + R64_KEYS - 1) / R64_KEYS : 0;  // sub-tiles

    // ---- tile movement: global -> LDS directly ---------------------------------------------------------------------
    // Wavefront w moves groups w, w + 4, w + 8, w + 12 of a tile: lane i of a load fetches row 16 (i / 16) + group,
    // 16-byte column i % 16 (a column in the padding of the head dim reads from beyond the buffer, i.e. zeros).
    const uint16_t *kg = (const uint16_t *)p.k + b * p.ks[0] + g * p.ks[1];
    const uint16_t *vg = (const uint16_t *)p.v + b * p.vs[0] + g * p.vs[1];
    const int krow_bytes = (int)p.ks[2] * 2, vrow_bytes = (int)p.vs[2] * 2;
    auto descriptor = [&](const uint16_t *base, int row_bytes) __attribute__((always_inline)) {
        const uint64_t ptr = (uint64_t)base;
        return uint4_t{(uint32_t)ptr, (uint32_t)(ptr >> 32) & 0xffffu, (uint32_t)((key_end - 1) * row_bytes + hd * 2),
                       0x00020000u};
    };
    const uint4_t krs = descriptor(kg, krow_bytes), vrs = descriptor(vg, vrow_bytes);
    const bool col_ok = (lane & 15) * 8 < hd;
    const int gofs_k = col_ok ? (16 * (lane >> 4) + wave) * krow_bytes + (lane & 15) * 16 : 0x7ffffff0;
    const int gofs_v = col_ok ? (16 * (lane >> 4) + wave) * vrow_bytes + (lane & 15) * 16 : 0x7ffffff0;
    const int lds0 = (int)(uint32_t)(uintptr_t)lds_base;
    // pieces [j_lo, j_hi) of LDS tile `tile` (a tile that starts beyond the key axis is never used: the offset is
    // clamped so it stays inside 32 bits)
    auto issue_loads = [&](const uint4_t rs, int gofs, int row_bytes, int tile, int lbase, int lstep, int j_lo, int j_hi)
                           __attribute__((always_inline)) {
        const int soff = __builtin_amdgcn_readfirstlane(min(j_begin + tile * R64_TILE, p.Skv) * row_bytes);
        lbase = __builtin_amdgcn_readfirstlane(lbase + lds0);
        // written as assembly on purpose: the compiler would otherwise make every later LDS read of this wavefront
        // wait for these loads, whose data is not due before a later barrier
#pragma unroll
        for (int j = j_lo; j < j_hi; j++)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :
                         : "s"(lbase + j * lstep), "v"(gofs), "s"(rs), "s"(soff + 4 * j * row_bytes)
                         : "memory", "m0");
    };
    // one tile load inside the loop: LDS address and buffer offset are formed inside the statement (the offset's add
    // also fills the wait state the LDS address register needs before the load)
    auto issue_one = [&](const uint4_t rs, int gofs, int lds_base_at, auto lds_step, int soff_base, int soff_step)
                         __attribute__((always_inline)) {
        int soff;
        asm volatile("s_add_u32 m0, %1, %2\n\ts_add_u32 %0, %3, %4\n\tbuffer_load_dwordx4 %5, %6, %0 offen lds"
                     : "=&s"(soff)
                     : "s"(lds_base_at), "n"(decltype(lds_step)::value), "s"(soff_base), "s"(soff_step), "v"(gofs), "s"(rs)
                     : "memory", "m0", "scc");
    };
    const int step4_k = 4 * krow_bytes, step4_v = 4 * vrow_bytes;
    auto k_stage = [&](int tile) __attribute__((always_inline)) { return (tile & (R64_NK - 1)) * R64_K_BYTES; };
    auto v_stage = [&](int tile) __attribute__((always_inline)) { return R64_V_AT + (tile & (R64_NV - 1)) * R64_V_BYTES; };
    if (ntiles > 0) {  // what the iterations before the first would have issued; the Q fetch below overlaps them
        issue_loads(krs, gofs_k, krow_bytes, 0, k_stage(0) + wave * KG, 4 * KG, 0, 4);
        issue_loads(vrs, gofs_v, vrow_bytes, 0, v_stage(0) + wave * VG, 4 * VG, 0, 4);
        issue_loads(krs, gofs_k, krow_bytes, 1, k_stage(1) + wave * KG, 4 * KG, 0, 4);
        issue_loads(vrs, gofs_v, vrow_bytes, 1, v_stage(1) + wave * VG, 4 * VG, 0, 4);
    }

    // Q^T operands: Q[query][16 kb + 8 h2 .. +8] of both row blocks, kept in registers for the whole kernel
    vec8 qreg[RB][KB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        const uint16_t *qp = (const uint16_t *)p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)qrow[rb] * p.qs[2];
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
            uint4_t raw = {0, 0, 0, 0};
            if (16 * kb + 8 * h2 < hd) raw = *(const uint4_t *)(qp + 16 * kb + 8 * h2);
            qreg[rb][kb] = __builtin_bit_cast(vec8, raw);
        }
    }

    float16_t o[RB][DB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[rb][db][r] = 0.0f;
    // m: the row's reference exponent in units of the S^T accumulators; nmr = -m * rr.  While the row has seen no key m
    // is -inf and nmr +inf, which sends the first tile with a visible key through the branch that sets m.
    float m[RB], l[RB], nmr[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) m[rb] = -INFINITY, l[rb] = 0.0f, nmr[rb] = INFINITY;

    // LDS operands in flight: the K operand slices of an S^T (the first half read during the block before), V's two
    // contraction slices, read one block apart.  Every operand feeds the matrix instructions of both row blocks.
    uint4_t ka[KB];
    uint4_t va[2][DB];
    // Scores and probabilities of the sub-tiles in flight, by the sub-tile's parity: while the matrix pipe writes
    // S^T(t + 1) the vector ALU reads S^T(t), and while it reads P(t - 1) the vector ALU writes P(t).
    float16_t sc[2][RB];
    uint32_t pk[2][RB][8];   // packed pairs in the matrix instruction's operand order
    const int klane = (ln & 15) * KG + (ln >> 4) * ROWB + h2 * 16;
    const int i16 = lane & 15, bl = (lane & 31) >> 4;
    const int vlane = (4 * h2 + (i16 >> 2)) * VG + (16 * bl + 4 * (i16 & 3)) * 2;
    // one address register per sub-tile and tensor: the reads of a sub-tile differ by immediate offsets only
    auto k_addr = [&](int t) __attribute__((always_inline)) {
        int base = k_stage(t >> 1) + (t & 1) * 2 * ROWB + klane;
        asm volatile("" : "+v"(base));
        return base;
    };
    auto v_addr = [&](int t) __attribute__((always_inline)) {
        int base = v_stage(t >> 1) + (t & 1) * 2 * ROWB + vlane;
        asm volatile("" : "+v"(base));
        return base;
    };
    auto read_k = [&](int base, int kb) __attribute__((always_inline)) { ka[kb] = *R64_LDS(uint4_t, base + kb * 32); };
    auto read_v = [&](int base, int kk, int db) __attribute__((always_inline)) {
        // contraction slice kk: keys 16 kk + 4 h2 + {0..3} and + 8
        const int addr = base + kk * ROWB + db * 64;
        const short4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(R64_LDS(short4_t, addr));
        const short4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(R64_LDS(short4_t, addr + 8 * VG));
        const uint2_t u0 = __builtin_bit_cast(uint2_t, a0), u1 = __builtin_bit_cast(uint2_t, a1);
        va[kk][db] = uint4_t{u0[0], u0[1], u1[0], u1[1]};
    };
    // The LDS operands belong in the accumulation half of the register file, where the reads can put them and the
    // matrix instructions take them from: the other half is for what the vector ALU touches.
    auto acc_half = [&](uint4_t &x) __attribute__((always_inline)) {
        asm("" : "+a"(x));
        return __builtin_bit_cast(vec8, x);
    };
    // probabilities of a tile against the reference nm (= -m * rr); returns this lane's sum
    auto probabilities = [&](const float (&s)[16], uint32_t (&pkr)[8], float nm) __attribute__((always_inline)) {
        float ts = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], rr, nm));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r + 1], rr, nm));
            pkr[r >> 1] = R64Mma<T>::pack2(p0, p1);
            ts += p0 + p1;
        }
        return ts;
    };
    // One sixteenth of a row block's softmax, placed beside a matrix instruction: the exponential of element s; the sum
    // takes the element before and the pair before that is packed (in their own step both would wait for the
    // exponential to leave its pipe).  softmax_rest: what the last step leaves.
    float pe[16];
    auto softmax_step = [&](const float16_t &s_in, uint32_t (&pkr)[8], float nm, float &ts, int s) __attribute__((always_inline)) {
        pe[s] = __builtin_amdgcn_exp2f(__builtin_fmaf(s_in[s], rr, nm));
        if (s >= 1) {
            ts += pe[s - 1];
            asm volatile("" : "+v"(ts));  // (the sum advances in its step, not in a chain behind the block)
        }
        if (s >= 2 && (s & 1) == 0) {
            pkr[(s - 2) >> 1] = R64Mma<T>::pack2(pe[s - 2], pe[s - 1]);
            asm volatile("" : "+v"(pkr[(s - 2) >> 1]));
        }
    };
    auto softmax_rest = [&](uint32_t (&pkr)[8], float &ts) __attribute__((always_inline)) {
        ts += pe[15];
        pkr[7] = R64Mma<T>::pack2(pe[14], pe[15]);
        asm volatile("" : "+v"(pkr[7]));
    };

    // Block B of sub-tile u (parity PAR = u & 1, ODD = the iteration's second half): O^T += V(u)^T . P(u)^T, steps
    // (kk, db, rb).  Beside it: the second contraction slice of V(u) leaves the LDS in the first eight steps, the first
    // operands of K(u + 2) and the first slice of V(u + 1) in the last eight; the first row block of sub-tile u + 1
    // becomes probabilities, one score per step; four tile loads are issued, one every four steps: K tile T + 2 in the
    // iteration's first half, V tile T + 2 in its second, into stages whose last readers are a barrier behind.
    auto block_b = [&](int u, auto par_c, auto odd_c, auto softmax_c, float &ts0) __attribute__((always_inline)) {
        constexpr int PAR = decltype(par_c)::value;
        constexpr bool ODD = decltype(odd_c)::value, SOFTMAX = decltype(softmax_c)::value;
        __builtin_amdgcn_sched_barrier(0);
        const int vbase = v_addr(u);
        const int kbase = k_addr(u + 2);
        const int vnext = v_addr(u + 1);
        const int tile = ((u + 1) >> 1) + 2;
        const int row_bytes = ODD ? vrow_bytes : krow_bytes;
        const int soff = __builtin_amdgcn_readfirstlane(min(j_begin + tile * R64_TILE, p.Skv) * row_bytes);
        const int lds_at = __builtin_amdgcn_readfirstlane(lds0 + (ODD ? v_stage(tile) + wave * VG : k_stage(tile) + wave * KG));
        constexpr int LSTEP = 4 * (ODD ? VG : KG);
        const int gstep = ODD ? step4_v : step4_k;
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
#pragma unroll
            for (int db = 0; db < DB; db++) {
#pragma unroll
                for (int rb = 0; rb < RB; rb++) {
                    const uint4_t braw = {pk[PAR][rb][4 * kk], pk[PAR][rb][4 * kk + 1], pk[PAR][rb][4 * kk + 2], pk[PAR][rb][4 * kk + 3]};
                    const vec8 bop = __builtin_bit_cast(vec8, braw);
                    // (the first slice's operands were read in the block before: the register allocator places them;
                    // the second slice's are read and used inside this block)
                    o[rb][db] = R64Mma<T>::mfma(kk == 0 ? __builtin_bit_cast(vec8, va[0][db]) : acc_half(va[1][db]), bop, o[rb][db]);
                    if (kk == 0 && rb == 0) read_v(vbase, 1, db);
                    if (kk == 1 && rb == 0) read_k(kbase, db);
                    if (kk == 1 && rb == 1) read_v(vnext, 0, db);
                    const int s = 8 * kk + 2 * db + rb;
                    if (s == 0) issue_one(ODD ? vrs : krs, ODD ? gofs_v : gofs_k, lds_at, std::integral_constant<int, 0>{}, soff, 0);
                    if (s == 4) issue_one(ODD ? vrs : krs, ODD ? gofs_v : gofs_k, lds_at, std::integral_constant<int, LSTEP>{}, soff, gstep);
                    if (s == 8) issue_one(ODD ? vrs : krs, ODD ? gofs_v : gofs_k, lds_at, std::integral_constant<int, 2 * LSTEP>{}, soff, 2 * gstep);
                    if (s == 12) issue_one(ODD ? vrs : krs, ODD ? gofs_v : gofs_k, lds_at, std::integral_constant<int, 3 * LSTEP>{}, soff, 3 * gstep);
                    if (SOFTMAX) softmax_step(sc[PAR ^ 1][0], pk[PAR ^ 1][0], nmr[0], ts0, s);
                    // scheduling groups: 0x008 matrix instruction, 0x100 LDS read
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        if (SOFTMAX) softmax_rest(pk[PAR ^ 1][0], ts0);
    };
    // Block A of sub-tile t (parity PAR): S^T(t + 1) on the matrix pipe, steps (kb, rb), first operands in ka; beside it
    // the second row block of sub-tile t becomes probabilities and the rest of K(t + 1)'s operands leave the LDS.
    auto block_a = [&](int t, auto par_c, float &ts1) __attribute__((always_inline)) {
        constexpr int PAR = decltype(par_c)::value;
        __builtin_amdgcn_sched_barrier(0);
        const int kbase = k_addr(t + 1);
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                if (kb == 0) R64Mma<T>::mfma_first_v(sc[PAR ^ 1][rb], ka[kb], qreg[rb][kb]);
                else R64Mma<T>::mfma_v(sc[PAR ^ 1][rb], ka[kb], qreg[rb][kb]);
                if (rb == 0 && kb + KB / 2 < KB) read_k(kbase, kb + KB / 2);
                softmax_step(sc[PAR][1], pk[PAR][1], nmr[1], ts1, 2 * kb + rb);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        softmax_rest(pk[PAR][1], ts1);
    };
    // The scores of sub-tile t outside the rows' intervals become -inf before the softmax reads them (element r is key
    // j0 + 8 (r / 4) + 4 h2 + r % 4); a sub-tile none of the wavefront's rows sees (the workgroup's other wavefronts do)
    // is all -inf.  Runs right behind the matrix instructions that wrote the scores: those are issued from inline
    // assembly, so the wait states a vector instruction owes them are written out here.
    auto mask_scores = [&](int t, auto par_c) __attribute__((always_inline)) {
        constexpr int PAR = decltype(par_c)::value;
        const int j0 = j_begin + t * R64_KEYS;
        if (__builtin_expect(!(j0 >= full_lo_w && j0 + R64_KEYS <= full_hi_w), 0)) {
            asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
            if (j0 >= hi_w || j0 + R64_KEYS <= lo_w) {
#pragma unroll
                for (int rb = 0; rb < RB; rb++)
#pragma unroll
                    for (int r = 0; r < 16; r++) sc[PAR][rb][r] = -INFINITY;
            } else {
#pragma unroll
                for (int rb = 0; rb < RB; rb++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int key = j0 + 8 * (r >> 2) + 4 * h2 + (r & 3);
                        sc[PAR][rb][r] = (key >= klo[rb] && key < khi[rb]) ? sc[PAR][rb][r] : -INFINITY;
                    }
            }
        }
    };
    // After a sub-tile's probabilities have been formed: a lane's sum not at most 2^15 (which also catches the +inf and
    // NaN a row without a reference produces) means some row of the wavefront needs its reference moved.  Every row's
    // reference moves to at least the tile's maximum, what the row has accumulated is rescaled if some row's reference
    // did move, and the tile's probabilities are formed again.
    auto settle = [&](auto par_c, float (&ts)[RB]) __attribute__((always_inline)) {
        constexpr int PAR = decltype(par_c)::value;
        if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(ts[0] <= 32768.0f) || !(ts[1] <= 32768.0f)) != 0, 0)) {
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                float s[16];
#pragma unroll
                for (int r = 0; r < 16; r++) s[r] = sc[PAR][rb][r];
                float mx = s[0];
#pragma unroll
                for (int r = 1; r < 16; r++) mx = fmaxf(mx, s[r]);
                mx = r64_half_swap_max(mx);
                const float m_new = fmaxf(m[rb], mx);
                const float corr = (m[rb] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f((m[rb] - m_new) * rr);
                if (__builtin_amdgcn_ballot_w64(m[rb] != -INFINITY && m_new != m[rb]) != 0) {
                    // (element by element where it lives, in the accumulation half of the register file: written as
                    // arithmetic the compiler copies all of O^T out ahead of the branch, on the path of every sub-tile)
#pragma unroll
                    for (int db = 0; db < DB; db++)
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            float tmp;
                            asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 %0, %1"
                                         : "+a"(o[rb][db][r]), "=&v"(tmp)
                                         : "v"(corr));
                        }
                    asm volatile("s_nop 7" ::: "memory");  // before a matrix instruction takes them as its C operand
                }
                m[rb] = m_new;
                l[rb] *= corr;
                nmr[rb] = (m[rb] == -INFINITY) ? INFINITY : -m[rb] * rr;
                ts[rb] = probabilities(s, pk[PAR][rb], (m[rb] == -INFINITY) ? 0.0f : nmr[rb]);
            }
        }
#pragma unroll
        for (int rb = 0; rb < RB; rb++) l[rb] += ts[rb];
    };
    using c0 = std::integral_constant<int, 0>;
    using c1 = std::integral_constant<int, 1>;

    if (ntiles > 0) {
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int kb = 0; kb < KB; kb++) qreg[rb][kb] = R64Mma<T>::scaled(qreg[rb][kb], pw);
        // "Sub-tile -1", whose P . V the first iteration runs like any other: probabilities and V operands of zero (the
        // V stage of tile 3, which nothing has been loaded into yet, is cleared for its second contraction slice).
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int i = 0; i < 8; i++) pk[1][rb][i] = 0;
#pragma unroll
        for (int db = 0; db < DB; db++) va[0][db] = uint4_t{0, 0, 0, 0};
        for (int c = tid; c < R64_V_BYTES / 16; c += 256) *R64_LDS(uint4_t, v_stage(3) + 16 * c) = uint4_t{0, 0, 0, 0};
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");  // K tile 0 and V tile 0 have landed
        lds_barrier();
        {
            const int kbase = k_addr(0);
#pragma unroll
            for (int kb = 0; kb < KB; kb++) read_k(kbase, kb);
#pragma unroll
            for (int kb = 0; kb < KB; kb++)
#pragma unroll
                for (int rb = 0; rb < RB; rb++)
                    if (kb == 0) R64Mma<T>::mfma_first_v(sc[0][rb], ka[kb], qreg[rb][kb]);
                    else R64Mma<T>::mfma_v(sc[0][rb], ka[kb], qreg[rb][kb]);
        }
        mask_scores(0, c0{});
        // Iteration T, sub-tiles 2 T and 2 T + 1: P . V of sub-tile 2 T - 1 beside the first half of sub-tile 2 T's
        // softmax, S^T of 2 T + 1 beside the second half; then the same one sub-tile on.  At its top all of this
        // wavefront's tile loads but the last four have landed and the barrier publishes them.  The last four are V tile
        // T + 1's, first read in the next iteration; K tile T + 1, issued in the first half of the last iteration, is
        // read in the second half of this one and must be among those waited for.  (No wait for the wavefront's LDS
        // reads at the barrier: nothing is loaded into a stage they can still be reading before the next barrier.)
        const int npairs = (ntiles + 1) >> 1;
        for (int tt = 0; tt < npairs; tt++) {
            const int t = 2 * tt;
            float ts[RB] = {0.0f, 0.0f};
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("s_waitcnt vmcnt(4)\n\ts_barrier" ::: "memory");
            block_b(t - 1, c1{}, std::false_type{}, std::true_type{}, ts[0]);
            block_a(t, c0{}, ts[1]);
            settle(c0{}, ts);
            mask_scores(t + 1, c1{});
            ts[0] = ts[1] = 0.0f;
            block_b(t, c0{}, std::true_type{}, std::true_type{}, ts[0]);
            block_a(t + 1, c1{}, ts[1]);
            settle(c1{}, ts);
            mask_scores(t + 2, c0{});
        }
        __builtin_amdgcn_sched_barrier(0);
        float unused = 0.0f;
        // (what it reads beside the matrix instructions is not used; the loads it issues fetch nothing that is read)
        block_b(2 * npairs - 1, c1{}, std::false_type{}, std::false_type{}, unused);
    }

    // the epilogue reuses the tile buffers: no tile load may still be on its way into them
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
    // ---- epilogue: out[query][dim] = O^T[dim][query] / l (no visible key: NaN like the reference's 0 / 0) -----------
    // transposed through a wavefront-private slice of the LDS so that every global store is a 16-byte piece of a
    // contiguous row; 32 rows per round for 2-byte outputs, 16 for f32
    constexpr int SLICE = 32 * (D * 2 + 16);
    static_assert(4 * SLICE <= R64_LDS_BYTES, "epilogue staging exceeds the tile buffers");
    const bool out_f32 = p.out_f32 != 0;
    const int esz = out_f32 ? 4 : 2;
    const int pitch = D * esz + 16;
    auto wbase = lds_base + wave * SLICE;
    const int rounds = out_f32 ? 2 : 1;
    const int rows_per_round = 32 / rounds;
    const int cpr = hd * esz / 16;
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        const float l_tot = r64_half_swap_sum(l[rb]);
        const float inv = 1.0f / l_tot;
        const bool dead = l_tot == 0.0f;
        if (out_vec) {
            for (int rd = 0; rd < rounds; rd++) {
                const int row_lo_ = rd * rows_per_round;
                if (ln >= row_lo_ && ln < row_lo_ + rows_per_round) {
#pragma unroll
                    for (int db = 0; db < DB; db++)
#pragma unroll
                        for (int rq = 0; rq < 4; rq++) {
                            float v4[4];
#pragma unroll
                            for (int e = 0; e < 4; e++) v4[e] = dead ? __builtin_nanf("") : o[rb][db][4 * rq + e] * inv;
                            const int dim = 32 * db + 8 * rq + 4 * h2;
                            if (out_f32) {
                                *(__attribute__((address_space(3))) float4_t *)(wbase + (ln - row_lo_) * pitch + dim * 4) =
                                    float4_t{v4[0], v4[1], v4[2], v4[3]};
                            } else {
                                const uint2_t pk2 = {R64Mma<T>::pack2(v4[0], v4[1]), R64Mma<T>::pack2(v4[2], v4[3])};
                                *(__attribute__((address_space(3))) uint2_t *)(wbase + ln * pitch + dim * 2) = pk2;
                            }
                        }
                }
                wave_lds_sync();
                for (int c = lane; c < rows_per_round * cpr; c += 64) {
                    const int row = c / cpr, col = c % cpr;
                    const int qr = qw0 + 32 * rb + row_lo_ + row;
                    if (qr < p.Sq) {
                        const uint4_t val = *(__attribute__((address_space(3))) uint4_t *)(wbase + row * pitch + col * 16);
                        const int64_t eidx = b * p.os[0] + h * p.os[1] + (int64_t)qr * p.os[2];
                        *(uint4_t *)((char *)p.out + eidx * esz + col * 16) = val;
                    }
                }
                wave_lds_sync();
            }
        } else if (query[rb] < p.Sq) {
            const int64_t obase = b * p.os[0] + h * p.os[1] + (int64_t)query[rb] * p.os[2];
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int dim = 32 * db + 8 * (r >> 2) + 4 * h2 + (r & 3);
                    if (dim >= hd) continue;
                    const float val = dead ? __builtin_nanf("") : o[rb][db][r] * inv;
                    if (p.out_f32) ((float *)p.out)[obase + dim * p.os[3]] = val;
                    else ((T *)p.out)[obase + dim * p.os[3]] = from_float<T>(val);
                }
        }
    }
}

template <typename T>
int launch_rows64_t(const AttnParams &p, hipStream_t stream) {
    const int nqb = (p.Sq + R64_BM - 1) / R64_BM;
    const long blocks = (long)nqb * p.B * p.H;
    if (blocks > 0x7fffffffL) {
        set_error("prefill: too many workgroups (%ld)", blocks);
        return FHIP_ERR_UNSUPPORTED;
    }
    // rows of the output can be written in 16-byte pieces when they are contiguous and aligned
    const int oeb = p.out_f32 ? 4 : 2;
    int out_vec = p.os[3] == 1 && ((uintptr_t)p.out % 16 == 0);
    for (int i = 0; i < 3; i++)
        if ((p.os[i] * oeb) % 16 != 0) out_vec = 0;
    FHIP_LAUNCH_MAIN((prefill_mfma_rows64_kernel<T>), dim3((unsigned)blocks), dim3(256), stream, p, p, nqb, out_vec);
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

}  // namespace

// The calls this form can run: head_dim 128 and a scale whose power-of-two part Q can carry without leaving the 16-bit
// type's normal range (keys are never split over workgroups, heads never packed).
bool prefill_mfma_rows64_takes(int D, float scale) {
    const float scale2 = scale * R64_LOG2E;
    return D == R64_D && scale2 >= 0.00390625f && scale2 < 2.0f;
}

int launch_prefill_mfma_rows64(const AttnParams &p, fhip_dtype dtype, hipStream_t stream) {
    if (dtype == FHIP_F16) return launch_rows64_t<half_t>(p, stream);
    if (dtype == FHIP_BF16) return launch_rows64_t<bf16_t>(p, stream);
    set_error("prefill MFMA kernel takes f16/bf16 only");
    return FHIP_ERR_UNSUPPORTED;
}

}  // namespace fhip
