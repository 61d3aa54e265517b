// Prefill attention for f16 / bf16 at head dims above 192 (Gemma-3's key length is 256) on the gfx950 matrix cores:
// every call at these head dims but those of up to 64 query rows whose keys are split over workgroups or whose heads
// are packed (a few new rows on a long cache, attn_prefill_mfma_wide.hip).
//
// At this head dim Q and O^T of 32 query rows are 192 registers of a wavefront, so two wavefronts per SIMD can only
// hold 16 rows each (prefill_mfma_wide_kernel), and every K and V operand a wavefront reads from LDS then feeds a
// single 16x16x32 matrix instruction: the CU's LDS has to deliver 256 bytes per clock for the matrix pipes to be busy.
// Here a workgroup is FOUR wavefronts of 32 rows, one per SIMD with the whole register file (512 registers), on
// v_mfma_f32_32x32x16 with the arithmetic of the 256-row kernel (attn_prefill_mfma.hip): half the LDS bytes per matrix
// instruction.  With one wavefront per SIMD nothing overlaps unless the instruction stream itself interleaves it, so
// the loop is software-pipelined over the 32-key tiles.  Iteration t:
//   block B:  O^T += V(t-1)^T . P(t-1)^T on the matrix pipe; beside it the LDS hands over the rest of V(t-1)'s operands,
//             the first of K(t+1)'s and the first of V(t)'s, the scores S^T(t) move to where the vector ALU reads them,
//             and the tile loads of the iteration are issued
//   block A:  S^T(t+1) = K(t+1) . Q^T on the matrix pipe; beside it the vector ALU turns S^T(t) into probabilities and
//             the LDS hands over the rest of K(t+1)'s operands
// Each block is sixteen steps of one matrix instruction and what runs beside it, fenced so that the compiler keeps
// them apart (a lone wavefront issues in order: a matrix instruction leaves room for about four other instructions
// before the next one is due, and whatever is not placed beside one is paid for in full).  K and V tiles live in rings
// of four LDS stages each, loaded straight into LDS (no staging registers) two iterations ahead of their first
// reader; one workgroup barrier per iteration publishes what has landed.
//
// Softmax as in the 256-row kernel: Q carries the power-of-two part of scale * log2(e), the rest (rr in [1, 2))
// multiplies the scores in f32; a probability is exp2(fma(s, rr, -m * rr)) against the reference m the row already
// has, and m moves only when a lane's probabilities of a tile sum to more than 2^15.
// Masking is by interval (attn_bounds.h): analytic descriptors, key counts, the interval form of a mask tensor.
//
// Reference semantics: fusor-ml/fusor/src/composite/flash_attention.rs:141-199 with the f32 accumulation of 16-bit
// inputs of fusor-ml/core/src/composite/flash_attention.rs:186-203,323-327.
#include <type_traits>

#include "attn_bounds.h"
#include "common.h"
#include "device_utils.h"

namespace fhip {

namespace {

constexpr float R32_LOG2E = 1.4426950408889634f;
constexpr int R32_D = 256;     // the kernel's head dim: the call's, a multiple of 8, is padded with zeros up to it
constexpr int R32_BM = 128;    // query rows per workgroup
constexpr int R32_KEYS = 32;   // keys per tile
// LDS image of a 32-row tile, as in the 256-row kernel: rows in 16 groups of 2 (row r in group r % 16 at position
// r / 16), a group being what one wavefront-wide direct load writes (1 KB), and groups padded apart so that the 16
// rows a quarter-wavefront reads for the S^T operand fall 16 bytes apart modulo the 256-byte bank period (K) and the
// 4 rows x 64 bytes a half-wavefront reads with the transposing load fall 64 bytes apart (V).
constexpr int R32_ROWB = R32_D * 2;
constexpr int R32_KG = 2 * R32_ROWB + 16;
constexpr int R32_VG = 2 * R32_ROWB + 64;
constexpr int R32_K_BYTES = 16 * R32_KG;
constexpr int R32_V_BYTES = 16 * R32_VG;
constexpr int R32_NK = 4, R32_NV = 4;
constexpr int R32_V_AT = R32_NK * R32_K_BYTES;
constexpr int R32_LDS_BYTES = R32_V_AT + R32_NV * R32_V_BYTES;

#define R32_LDS(type, byte_off) ((__attribute__((address_space(3))) type *)(lds_base + (byte_off)))

template <typename T>
struct R32Mma;
template <>
struct R32Mma<half_t> {
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
struct R32Mma<bf16_t> {
    typedef bf16x8_t vec8;
    static __device__ __forceinline__ float16_t mfma(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
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

__device__ __forceinline__ float r32_half_swap_max(float x) {  // max of x with the value held by the lane 32 away
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float r32_half_swap_sum(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// SPLIT: the keys are split over workgroups (an instantiation of its own: the kernel sits at the edge of the register
// file, and the code of the split form costs the unsplit one spills inside its loop).
template <typename T, bool SPLIT>
__global__ __launch_bounds__(256, 1) void prefill_mfma_wide_rows32_kernel(AttnParams p, int nqb, int out_vec) {
    typedef typename R32Mma<T>::vec8 vec8;
    constexpr int D = R32_D, ROWB = R32_ROWB, KG = R32_KG, VG = R32_VG;
    __shared__ __attribute__((aligned(16))) char smem[R32_LDS_BYTES];
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
    const int nks = SPLIT ? max(p.pf_nsplit, 1) : 1;
    const int ksplit = SPLIT ? blockIdx.x % nks : 0;  // which share of the keys
    const int id = SPLIT ? blockIdx.x / nks : blockIdx.x;
    const int qb = nqb - 1 - id / bh_count;
    const int rem = id % bh_count;
    const int b = rem / p.H;
    int h = rem % p.H;
    if ((p.H & 7) == 0) h = (h & 7) * (p.H >> 3) + (h >> 3);
    const int g = h / p.G;
    // rows of a tile beyond the sequence's own keys read as zero (the buffers end there)
    int key_end = p.kv_lens ? min(p.Skv, max(p.kv_lens[b], 1)) : p.Skv;
    if (p.analytic && p.causal) key_end = (int)min((int64_t)key_end, max(p.q_pos_offset + p.Sq, (int64_t)1));

    const int q0 = qb * R32_BM, qw0 = q0 + 32 * wave;
    const int query = qw0 + ln;
    RowBounds rb = row_bounds(p, b, q0, R32_BM, qw0, lane);
    if (SPLIT) {  // a few query blocks on a long cache: this workgroup takes one share of the keys
        const int c_lo = ksplit * p.pf_chunk, c_hi = c_lo + p.pf_chunk;
        rb.lo_wg = max(rb.lo_wg, c_lo), rb.hi_wg = min(rb.hi_wg, c_hi);
        rb.full_lo_w = max(rb.full_lo_w, c_lo), rb.full_hi_w = min(rb.full_hi_w, c_hi);
        rb.klo = max(rb.klo, c_lo), rb.khi = min(rb.khi, c_hi);
    }
    const int klo = rb.klo, khi = rb.khi;
    const int lo_wg = __builtin_amdgcn_readfirstlane(rb.lo_wg), hi_wg = __builtin_amdgcn_readfirstlane(rb.hi_wg);
    const int full_lo_w = __builtin_amdgcn_readfirstlane(rb.full_lo_w), full_hi_w = __builtin_amdgcn_readfirstlane(rb.full_hi_w);
    const int qrow = min(query, p.Sq - 1);

    const float scale2 = p.scale * R32_LOG2E;
    // scale2 = pw * rr with pw a power of two and rr in [1, 2): Q takes pw (exact), rr multiplies every score in f32
    const float pw = __uint_as_float(__float_as_uint(scale2) & 0x7F800000u);
    const float rr = scale2 / pw;

    const int j_begin = (lo_wg / R32_KEYS) * R32_KEYS;
    const int ntiles = hi_wg > j_begin ? (hi_wg - j_begin + R32_KEYS - 1) / R32_KEYS : 0;

    // ---- tile movement: global -> LDS directly ---------------------------------------------------------------------
    // Wavefront w moves groups w, w + 4, w + 8, w + 12 of a tile: lane i of a load fetches row 16 (i / 32) + group,
    // 16-byte column i % 32 (a column in the padding of the head dim reads from beyond the buffer, i.e. zeros).
    const uint16_t *kg = (const uint16_t *)p.k + b * p.ks[0] + g * p.ks[1];
    const uint16_t *vg = (const uint16_t *)p.v + b * p.vs[0] + g * p.vs[1];
    const int krow_bytes = (int)p.ks[2] * 2, vrow_bytes = (int)p.vs[2] * 2;
    auto descriptor = [&](const uint16_t *base, int row_bytes) __attribute__((always_inline)) {
        const uint64_t ptr = (uint64_t)base;
        return uint4_t{(uint32_t)ptr, (uint32_t)(ptr >> 32) & 0xffffu, (uint32_t)((key_end - 1) * row_bytes + hd * 2),
                       0x00020000u};
    };
    const uint4_t krs = descriptor(kg, krow_bytes), vrs = descriptor(vg, vrow_bytes);
    const bool col_ok = (lane & 31) * 8 < hd;
    const int gofs_k = col_ok ? (16 * (lane >> 5) + wave) * krow_bytes + (lane & 31) * 16 : 0x7ffffff0;
    const int gofs_v = col_ok ? (16 * (lane >> 5) + wave) * vrow_bytes + (lane & 31) * 16 : 0x7ffffff0;
    const int lds0 = (int)(uint32_t)(uintptr_t)lds_base;
    auto issue_loads = [&](const uint4_t rs, int gofs, int row_bytes, int tile, int lbase, int lstep)
                           __attribute__((always_inline)) {
        // (a tile that starts beyond the key axis is never used: the offset is clamped so it stays inside 32 bits)
        const int soff = __builtin_amdgcn_readfirstlane(min(j_begin + tile * R32_KEYS, p.Skv) * row_bytes);
        lbase = __builtin_amdgcn_readfirstlane(lbase + lds0);
        // written as assembly on purpose: the compiler would otherwise make every later LDS read of this wavefront
        // wait for these loads, whose data is not due before a later barrier
#pragma unroll
        for (int j = 0; j < 4; j++)
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
    auto issue_piece_k = [&](int j, int lds_at, int soff) __attribute__((always_inline)) {
        if (j == 0) issue_one(krs, gofs_k, lds_at, std::integral_constant<int, 0>{}, soff, 0);
        else if (j == 1) issue_one(krs, gofs_k, lds_at, std::integral_constant<int, 4 * KG>{}, soff, step4_k);
        else if (j == 2) issue_one(krs, gofs_k, lds_at, std::integral_constant<int, 8 * KG>{}, soff, 2 * step4_k);
        else issue_one(krs, gofs_k, lds_at, std::integral_constant<int, 12 * KG>{}, soff, 3 * step4_k);
    };
    auto issue_piece_v = [&](int j, int lds_at, int soff) __attribute__((always_inline)) {
        if (j == 0) issue_one(vrs, gofs_v, lds_at, std::integral_constant<int, 0>{}, soff, 0);
        else if (j == 1) issue_one(vrs, gofs_v, lds_at, std::integral_constant<int, 4 * VG>{}, soff, step4_v);
        else if (j == 2) issue_one(vrs, gofs_v, lds_at, std::integral_constant<int, 8 * VG>{}, soff, 2 * step4_v);
        else issue_one(vrs, gofs_v, lds_at, std::integral_constant<int, 12 * VG>{}, soff, 3 * step4_v);
    };
    auto k_stage = [&](int t) __attribute__((always_inline)) { return (t & (R32_NK - 1)) * R32_K_BYTES; };
    auto v_stage = [&](int t) __attribute__((always_inline)) { return R32_V_AT + (t & (R32_NV - 1)) * R32_V_BYTES; };
    auto issue_k = [&](int tile) __attribute__((always_inline)) {
        issue_loads(krs, gofs_k, krow_bytes, tile, k_stage(tile) + wave * KG, 4 * KG);
    };
    auto issue_v = [&](int tile) __attribute__((always_inline)) {
        issue_loads(vrs, gofs_v, vrow_bytes, tile, v_stage(tile) + wave * VG, 4 * VG);
    };
    if (ntiles > 0) {  // what the iterations before the first would have issued; the Q fetch below overlaps them
        issue_k(0);
        issue_k(1);
        issue_v(0);
        issue_k(2);
        issue_v(1);
    }

    // Q^T operand: Q[query][16 kb + 8 h2 .. +8], kept in registers for the whole kernel
    vec8 qreg[D / 16];
    {
        const uint16_t *qp = (const uint16_t *)p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)qrow * p.qs[2];
#pragma unroll
        for (int kb = 0; kb < D / 16; kb++) {
            uint4_t raw = {0, 0, 0, 0};
            if (16 * kb + 8 * h2 < hd) raw = *(const uint4_t *)(qp + 16 * kb + 8 * h2);
            qreg[kb] = __builtin_bit_cast(vec8, raw);
        }
    }

    float16_t o[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.0f;
    // m: the row's reference exponent in units of the S^T accumulators; nmr = -m * rr.  While the row has seen no key m
    // is -inf and nmr +inf, which sends the first tile with a visible key through the branch that sets m.
    float m = -INFINITY, l = 0.0f, nmr = INFINITY;
    float16_t zero16;
#pragma unroll
    for (int r = 0; r < 16; r++) zero16[r] = 0.0f;

    // LDS operands in flight: the first / last eight K operand slices of an S^T take turns in ka (the first eight are
    // read during the block before, the last eight while the first are being used); V's two contraction slices are
    // read one block apart
    constexpr int PFK = 8;
    uint4_t ka[PFK];
    uint4_t va[2][D / 32];
    uint32_t pk[8];          // probabilities, packed pairs in the matrix instruction's operand order
    float16_t sn;            // S^T as the matrix instructions leave it
    float sx[16];            // the same once the vector ALU can read it
    const int klane = (ln & 15) * KG + (ln >> 4) * ROWB + h2 * 16;
    const int i16 = lane & 15, bl = (lane & 31) >> 4;
    const int vlane = (4 * h2 + (i16 >> 2)) * VG + (16 * bl + 4 * (i16 & 3)) * 2;
    // one address register per tile and tensor: the reads of a tile differ by immediate offsets only
    auto k_addr = [&](int tile) __attribute__((always_inline)) {
        int base = k_stage(tile) + klane;
        asm volatile("" : "+v"(base));
        return base;
    };
    auto v_addr = [&](int tile) __attribute__((always_inline)) {
        int base = v_stage(tile) + vlane;
        asm volatile("" : "+v"(base));
        return base;
    };
    auto read_k = [&](int base, int kb) __attribute__((always_inline)) { ka[kb % PFK] = *R32_LDS(uint4_t, base + kb * 32); };
    auto read_v = [&](int base, int kk, int db) __attribute__((always_inline)) {
        // contraction slice kk: keys 16 kk + 4 h2 + {0..3} and + 8
        const int addr = base + kk * ROWB + db * 64;
        const short4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(R32_LDS(short4_t, addr));
        const short4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(R32_LDS(short4_t, addr + 8 * VG));
        const uint2_t u0 = __builtin_bit_cast(uint2_t, a0), u1 = __builtin_bit_cast(uint2_t, a1);
        va[kk][db] = uint4_t{u0[0], u0[1], u1[0], u1[1]};
    };
    // The LDS operands belong in the accumulation half of the register file, where the reads can put them and the
    // matrix instructions take them from: the other half is for what the vector ALU touches (Q is read by every tile
    // and would otherwise be the one moved out and copied back before every matrix instruction).
    auto acc_half = [&](uint4_t x) __attribute__((always_inline)) {
        asm("" : "+a"(x));
        return __builtin_bit_cast(vec8, x);
    };
    // probabilities of a tile against the reference nm (= -m * rr); returns this lane's sum
    auto probabilities = [&](const float (&s)[16], float nm) __attribute__((always_inline)) {
        float ts = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], rr, nm));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r + 1], rr, nm));
            pk[r >> 1] = R32Mma<T>::pack2(p0, p1);
            ts += p0 + p1;
        }
        return ts;
    };

    // Both blocks are written as sixteen steps that nothing crosses: a matrix instruction first, then the LDS reads,
    // tile loads and vector work that run beside it (left to itself the scheduler issues the matrix instructions back
    // to back and the rest behind them, where nothing hides it).
    // Block B of tile u: O^T += V(u)^T . P(u)^T.  Beside it: the second contraction slice of V(u) leaves the LDS in the
    // first eight steps, the first operands of K(u + 2) and the first slice of V(u + 1) (for the next iteration's block
    // B: in block A, beside the exponentials, the transposing reads cost more) in the last eight; the scores of tile
    // u + 1 leave the accumulation half of the register file, one per step; this iteration's tile loads are issued, one
    // every other step: K(u + 4) into the stage K(u) left one iteration ago, V(u + 3) into the stage V(u - 1) left then.
    auto block_b = [&](int u) __attribute__((always_inline)) {
        __builtin_amdgcn_sched_barrier(0);
        const int vbase = v_addr(u);
        const int kbase = k_addr(u + 2);
        const int vnext = v_addr(u + 1);
        const int soff_k = __builtin_amdgcn_readfirstlane(min(j_begin + (u + 4) * R32_KEYS, p.Skv) * krow_bytes);
        const int soff_v = __builtin_amdgcn_readfirstlane(min(j_begin + (u + 3) * R32_KEYS, p.Skv) * vrow_bytes);
        const int lds_k = __builtin_amdgcn_readfirstlane(lds0 + k_stage(u + 4) + wave * KG);
        const int lds_v = __builtin_amdgcn_readfirstlane(lds0 + v_stage(u + 3) + wave * VG);
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            const uint4_t braw = {pk[4 * kk], pk[4 * kk + 1], pk[4 * kk + 2], pk[4 * kk + 3]};
            const vec8 bop = __builtin_bit_cast(vec8, braw);
#pragma unroll
            for (int db = 0; db < D / 32; db++) {
                // (the first slice's operands were read in the block before, across the loop's back edge: the register
                // allocator places them; the second slice's are read and used inside this block)
                o[db] = R32Mma<T>::mfma(kk == 0 ? __builtin_bit_cast(vec8, va[0][db]) : acc_half(va[1][db]), bop, o[db]);
                if (kk == 0) read_v(vbase, 1, db);
                else read_k(kbase, db);
                if (kk == 1) read_v(vnext, 0, db);
                if ((db & 1) == 0) {
                    if (kk == 0) issue_piece_k(db >> 1, lds_k, soff_k);
                    else issue_piece_v(db >> 1, lds_v, soff_v);
                }
                const int r = 8 * kk + db;
                sx[r] = sn[r];
                asm volatile("" : "+v"(sx[r]));
                // scheduling groups: 0x008 matrix instruction, 0x100 LDS read
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    // Block A of tile t: S^T(t + 1) on the matrix pipe (first operands in ka); beside it the probabilities of tile t
    // (scores in sx) and the rest of K(t + 1)'s operands.  Returns the lane's sum.
    auto block_a = [&](int t) __attribute__((always_inline)) {
        __builtin_amdgcn_sched_barrier(0);
        const int kbase = k_addr(t + 1);
        float ts = 0.0f;
        float pe[16];
#pragma unroll
        for (int kb = 0; kb < D / 16; kb++) {
            sn = R32Mma<T>::mfma(acc_half(ka[kb % PFK]), qreg[kb], kb == 0 ? zero16 : sn);
            if (kb + PFK < D / 16) read_k(kbase, kb + PFK);
            pe[kb] = __builtin_amdgcn_exp2f(__builtin_fmaf(sx[kb], rr, nmr));
            if (kb & 1) {
                // (formed here, in its step, not behind the branch that follows the block)
                pk[kb >> 1] = R32Mma<T>::pack2(pe[kb - 1], pe[kb]);
                asm volatile("" : "+v"(pk[kb >> 1]));
                ts += pe[kb - 1] + pe[kb];
            }
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        return ts;
    };

    if (ntiles > 0) {
#pragma unroll
        for (int kb = 0; kb < D / 16; kb++) qreg[kb] = R32Mma<T>::scaled(qreg[kb], pw);
        // "Tile -1", whose P . V the first iteration runs like any other: probabilities and V operands of zero (the
        // V stage of tile 3, which nothing has been loaded into yet, is cleared for its second contraction slice).
#pragma unroll
        for (int i = 0; i < 8; i++) pk[i] = 0;
#pragma unroll
        for (int db = 0; db < D / 32; db++) va[0][db] = uint4_t{0, 0, 0, 0};
        for (int c = tid; c < R32_V_BYTES / 16; c += 256) *R32_LDS(uint4_t, v_stage(3) + 16 * c) = uint4_t{0, 0, 0, 0};
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");  // K(0), K(1), V(0) have landed
        lds_barrier();
        {
            const int kbase = k_addr(0);
#pragma unroll
            for (int kb = 0; kb < PFK; kb++) read_k(kbase, kb);
#pragma unroll
            for (int kb = 0; kb < D / 16; kb++) {
                sn = R32Mma<T>::mfma(acc_half(ka[kb % PFK]), qreg[kb], kb == 0 ? zero16 : sn);
                if (kb + PFK < D / 16) read_k(kbase, kb + PFK);
            }
        }
        // iteration t: P . V of tile t - 1, then the probabilities of tile t beside S^T of tile t + 1.  At its top
        // all of this wavefront's tile loads but the eight of the last iteration have landed and the barrier
        // publishes them: K(t + 1) and V(t) among them, issued two iterations ago.  (No wait for the wavefront's LDS
        // reads at the barrier: those that can still be on their way are of V(t - 1), and nothing is loaded into
        // that stage before the next barrier.)
        for (int t = 0; t < ntiles; t++) {
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");
            block_b(t - 1);
            const int j0 = j_begin + t * R32_KEYS;
            if (__builtin_expect(!(j0 >= full_lo_w && j0 + R32_KEYS <= full_hi_w), 0)) {
                // element r is key j0 + 8 (r / 4) + 4 h2 + r % 4
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int key = j0 + 8 * (r >> 2) + 4 * h2 + (r & 3);
                    sx[r] = (key >= klo && key < khi) ? sx[r] : -INFINITY;
                }
            }
            float ts = block_a(t);
            // Not at most 2^15 (which also catches the +inf and NaN a row without a reference produces): some row of
            // the wavefront needs its reference moved.  Take the tile's maximum, move every row's reference to at
            // least that, rescale what the row has accumulated, and form the tile's probabilities again.
            if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(ts <= 32768.0f)) != 0, 0)) {
                float mx = sx[0];
#pragma unroll
                for (int r = 1; r < 16; r++) mx = fmaxf(mx, sx[r]);
                mx = r32_half_swap_max(mx);
                const float m_new = fmaxf(m, mx);
                const float corr = (m == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f((m - m_new) * rr);
                m = m_new;
                l *= corr;
#pragma unroll
                for (int db = 0; db < D / 32; db++)
#pragma unroll
                    for (int r = 0; r < 16; r++) o[db][r] *= corr;
                nmr = (m == -INFINITY) ? INFINITY : -m * rr;
                ts = probabilities(sx, (m == -INFINITY) ? 0.0f : nmr);
            }
            l += ts;
        }
        __builtin_amdgcn_sched_barrier(0);
        block_b(ntiles - 1);  // (what it reads beside the matrix instructions is not used; the loads it issues fetch nothing)
    }

    // the epilogue reuses the tile buffers: no tile load may still be on its way into them
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
    // ---- epilogue: out[query][dim] = O^T[dim][query] / l (no visible key: NaN like the reference's 0 / 0) -----------
    const float l_tot = r32_half_swap_sum(l);
    if (SPLIT) {
        // this share's state: O unnormalised as f32, then (m in base-2 exponent units, l); the merge kernel normalises
        if (query < p.Sq) {
            float *ws = p.partials + ((((int64_t)b * p.H + h) * p.Sq + query) * nks + ksplit) * p.pf_pitch;
#pragma unroll
            for (int db = 0; db < D / 32; db++)
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    const int dim = 32 * db + 8 * rq + 4 * h2;
                    if (dim < hd) *(float4_t *)(ws + dim) = float4_t{o[db][4 * rq], o[db][4 * rq + 1], o[db][4 * rq + 2], o[db][4 * rq + 3]};
                }
            if (h2 == 0) {
                ws[hd] = m * rr;
                ws[hd + 1] = l_tot;
            }
        }
        return;
    }
    const float inv = 1.0f / l_tot;
    const bool dead = l_tot == 0.0f;
    if (out_vec) {
        // transpose through a wavefront-private slice of the LDS so that every global store is a 16-byte piece of a
        // contiguous row; 32 rows per round for 2-byte outputs, 16 for f32
        constexpr int SLICE = 32 * (D * 2 + 16);
        static_assert(4 * SLICE <= R32_LDS_BYTES, "epilogue staging exceeds the tile buffers");
        const bool out_f32 = p.out_f32 != 0;
        const int esz = out_f32 ? 4 : 2;
        const int pitch = D * esz + 16;
        auto wbase = lds_base + wave * SLICE;
        const int rounds = out_f32 ? 2 : 1;
        const int rows_per_round = 32 / rounds;
        const int cpr = hd * esz / 16;
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
                            const uint2_t pk2 = {R32Mma<T>::pack2(v4[0], v4[1]), R32Mma<T>::pack2(v4[2], v4[3])};
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
                    const int64_t eidx = b * p.os[0] + h * p.os[1] + (int64_t)qr * p.os[2];
                    *(uint4_t *)((char *)p.out + eidx * esz + col * 16) = val;
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
                if (dim >= hd) continue;
                const float val = dead ? __builtin_nanf("") : o[db][r] * inv;
                if (p.out_f32) ((float *)p.out)[obase + dim * p.os[3]] = val;
                else ((T *)p.out)[obase + dim * p.os[3]] = from_float<T>(val);
            }
    }
}

template <typename T>
int launch_rows32_t(const AttnParams &p, hipStream_t stream) {
    const int nqb = (p.Sq + R32_BM - 1) / R32_BM;
    const long blocks = (long)nqb * p.B * p.H * (p.pf_nsplit > 1 ? p.pf_nsplit : 1);
    if (blocks > 0x7fffffffL) {
        set_error("prefill: too many workgroups (%ld)", blocks);
        return FHIP_ERR_UNSUPPORTED;
    }
    // rows of the output can be written in 16-byte pieces when they are contiguous and aligned
    const int oeb = p.out_f32 ? 4 : 2;
    int out_vec = p.os[3] == 1 && ((uintptr_t)p.out % 16 == 0);
    for (int i = 0; i < 3; i++)
        if ((p.os[i] * oeb) % 16 != 0) out_vec = 0;
    if (p.pf_nsplit > 1) FHIP_LAUNCH_MAIN((prefill_mfma_wide_rows32_kernel<T, true>), dim3((unsigned)blocks), dim3(256), stream, p, p, nqb, out_vec);
    else FHIP_LAUNCH_MAIN((prefill_mfma_wide_rows32_kernel<T, false>), dim3((unsigned)blocks), dim3(256), stream, p, p, nqb, out_vec);
    FHIP_HIP_CHECK(hipGetLastError());
    if (p.pf_nsplit > 1) return launch_prefill_merge(p, std::is_same<T, half_t>::value ? FHIP_F16 : FHIP_BF16, stream);
    return FHIP_OK;
}

}  // namespace

// The calls this form takes: head dims above 192 (padded with zeros up to 256: f16, 4096 x 4096 causal, 16 heads, head_dim
// 200 / 224 / 232 195 / 208 / 218 -> 155 / 160 / 161 us against the 16-row form; up to 192 a wavefront of that form holds
// 32 rows itself), no packed heads, keys split over workgroups only from 65 query rows on (f16, head_dim 256, 16 / 4
// heads, 128 rows on B8 x 8192 keys 263 -> 186 us, on B1 x 32768 keys 120 -> 102), and a scale whose power-of-two part Q
// can carry without leaving the 16-bit type's normal range.
bool prefill_mfma_rows32_takes(const AttnParams &p) {
    const float scale2 = p.scale * R32_LOG2E;
    // (keys split over workgroups: from 65 query rows on; up to 64 the 16-row kernel's 64-row and packed forms serve)
    return p.D > 192 && p.D <= R32_D && p.D % 8 == 0 && (p.pf_nsplit <= 1 || p.Sq > 64) && !p.pf_pack && scale2 >= 0.00390625f &&
           scale2 < 2.0f;
}

int launch_prefill_mfma_rows32(const AttnParams &p, fhip_dtype dtype, hipStream_t stream) {
    if (dtype == FHIP_F16) return launch_rows32_t<half_t>(p, stream);
    if (dtype == FHIP_BF16) return launch_rows32_t<bf16_t>(p, stream);
    set_error("prefill MFMA kernel takes f16/bf16 only");
    return FHIP_ERR_UNSUPPORTED;
}

}  // namespace fhip
