// Prefill attention for f16 / bf16 at head dims 160, 192, 224 and 256 (Gemma-3's key length is 256) on the gfx950
// matrix cores, and at every other multiple of 8 up to 256 that the 256-row kernel (64 / 96 / 128) does not take: the
// kernel's D is the head dim rounded up to a multiple of 32, the padding dims read as zero and are not written.
//
// The 256-row kernel of attn_prefill_mfma.hip keeps Q and O^T of 32 rows in a wavefront's registers with two wavefronts
// per SIMD; at these head dims that is 192 registers and more for the two alone.  Here a workgroup is eight wavefronts
// of 16 query rows, two per SIMD, and 128 query rows of one (batch, head) (four wavefronts of 16 rows and 64 query rows,
// two workgroups per CU, on small grids); the keys are walked in tiles of 32 that all wavefronts share through LDS,
// loaded straight into it (no staging registers) with the next two tiles on their way during the math.  Per tile and
// wavefront, on v_mfma_f32_16x16x32 with the query rows as blocks of 16 columns (the arithmetic of the split-KV decode
// kernel, attn_decode.hip; the template also holds a form with two column blocks per wavefront):
//   S^T[key][row]  = K . Q^T     A = K from LDS (one 16-byte read feeds every column block), B = Q in registers
//   scores scaled in f32 (scale * log2 e), masked by the row's visible interval, online softmax per column
//   O^T[dim][row] += V^T . P^T   A = V^T from row-major LDS with ds_read_b64_tr_b16, B = the probabilities
// Masks: the analytic descriptor, key counts, or the interval form of a mask tensor (attn_bounds.h); a mask tensor that
// is not made of intervals is served by the kernel queued behind this one, as for the other tiled kernels.
//
// Reference semantics: fusor-ml/fusor/src/composite/flash_attention.rs:141-199 with the f32 accumulation of 16-bit
// inputs of fusor-ml/core/src/composite/flash_attention.rs:186-203,323-327.
#include <type_traits>

#include "attn_bounds.h"
#include "common.h"
#include "device_utils.h"

namespace fhip {

namespace {

constexpr float PW_LOG2E = 1.4426950408889634f;
constexpr int PW_BM = 128;  // query rows per workgroup: four wavefronts of 32 rows or eight of 16 (64 on small grids)
constexpr int PW_KEYS = 32;           // keys per tile
constexpr float PW_RESCALE_SLACK = 8.0f;

#define PWLDS_PTR(type, byte_off) ((__attribute__((address_space(3))) type *)(lds_base + (byte_off)))

typedef uint32_t uint2w_t __attribute__((ext_vector_type(2)));

template <typename T>
struct WideMma;
template <>
struct WideMma<half_t> {
    typedef half8_t vec8;
    static __device__ __forceinline__ float4_t mfma(vec8 a, vec8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float x, float y) {
        half2_t h = {(half_t)x, (half_t)y};
        return __builtin_bit_cast(uint32_t, h);
    }
};
template <>
struct WideMma<bf16_t> {
    typedef bf16x8_t vec8;
    static __device__ __forceinline__ float4_t mfma(vec8 a, vec8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float x, float y) {
        typedef __bf16 bf16x2w_t __attribute__((ext_vector_type(2)));
        const bf16x2w_t h = {(__bf16)x, (__bf16)y};  // v_cvt_pk_bf16_f32: round to nearest even
        return __builtin_bit_cast(uint32_t, h);
    }
};

// max / sum over the four lanes l, l^16, l^32, l^48 (same column, the four key groups)
__device__ __forceinline__ float pw_quad_max(float x) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float pw_quad_sum(float x) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// PW_WAVES wavefronts of 16 * CB query rows.  <8, 1>: 128-row workgroups, one per CU; <8, 2>: 256-row workgroups (up to
// head_dim 192, where 32 rows fit a wavefront's half of the register file); <4, 1>: 64-row workgroups, two per CU, for
// grids that would leave CUs idle; <4, 2> (four wavefronts with the whole register file each) is not launched any more.
template <typename T, int D, int PW_WAVES, int CB>
__global__ __launch_bounds__(64 * PW_WAVES, PW_WAVES * CB >= 8 ? 1 : 2) void prefill_mfma_wide_kernel(AttnParams p, int nqb) {
    typedef typename WideMma<T>::vec8 vec8;
    constexpr int KP = D * 2 + 16;           // K tile row pitch (bytes): rows 4 banks apart
    constexpr int VP = D * 2 + 32;           // V tile row pitch (bytes): rows 8 banks apart
    constexpr int K_BYTES = PW_KEYS * KP;
    constexpr int V_BYTES = PW_KEYS * VP;
    // a tile is filled 1 KB at a time (see the tile movement below): each tensor's region is whole pieces
    constexpr int NIK = (K_BYTES + 1023) / 1024, NIV = (V_BYTES + 1023) / 1024;
    constexpr int V_AT = NIK * 1024;                  // where the V tile starts in a stage
    constexpr int STAGE = (NIK + NIV) * 1024;
    constexpr int KB = D / 32;               // contraction blocks of K . Q^T
    constexpr int NB = D / 16;               // 16-dim blocks of the output
    constexpr int BM = 16 * CB * PW_WAVES;   // query rows per workgroup (CB 16-column blocks per wavefront)
    // tiles in LDS: the one in use and the next two on their way; the two-per-CU form has room for one on its way only
    constexpr int NSTAGE = PW_WAVES * CB >= 8 ? 3 : 2;
    __shared__ __attribute__((aligned(16))) char smem[NSTAGE * STAGE];
    auto lds_base = (__attribute__((address_space(3))) char *)smem;

    if (p.iv_bad && *p.iv_bad == p.bad_tag) return;  // the mask is not made of intervals: the kernel behind takes the call
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int j = lane & 15;   // column inside a block
    const int q4 = lane >> 4;  // key group
    const int hd = p.D;        // the head dim itself: a multiple of 8, padded with zeros up to the kernel's D

    // workgroup -> (share of the keys, query block, batch, head): long (late) query blocks first
    // Packed form (at most 32 query rows, GQA group a multiple of 4; not for the 64-row workgroups): the workgroup's
    // wavefronts hold rows 0..31 of four query heads that share a KV head (wavefront w: head w % 4, and with eight
    // wavefronts rows 16 (w / 4) ...), so the K and V tiles it moves serve all four and a few new rows on a long cache
    // read the cache once per KV head, not once per query head.
    const int pack = (PW_WAVES * CB == 8) ? p.pf_pack : 0;
    const int heads = pack ? p.H / 4 : p.H;  // head units per batch entry
    const int bh_count = p.B * heads;
    const int nks = max(p.pf_nsplit, 1);
    const int ksplit = blockIdx.x % nks;  // which share of the keys (0 when the keys are not split over workgroups)
    const int id = blockIdx.x / nks;
    const int qb = nqb - 1 - id / bh_count;
    const int rem = id % bh_count;
    const int b = rem / heads;
    int h = rem % heads;
    // consecutive workgroups land on consecutive XCDs (id % 8), each with an L2 of its own: with H a multiple of 8 the
    // heads are dealt so that an XCD works on H / 8 neighbouring heads, i.e. on as few KV heads as possible
    if (pack) h = 4 * h + (wave & 3);
    else if ((p.H & 7) == 0) h = (h & 7) * (p.H >> 3) + (h >> 3);
    const int g = h / p.G;
    // Rows of a tile beyond the sequence's own keys (kv_lens below the view's length: a ragged batch in one cache
    // allocation) read as zero (the buffers end there): what such rows hold, NaN included, must not reach the result as 0 x NaN in P . V.
    // (likewise the rows behind the last query's own position when the call says where its rows stand inside a longer
    // cache view: a causal descriptor with q_pos_offset + Sq below the view's length)
    int key_end = p.kv_lens ? min(p.Skv, max(p.kv_lens[b], 1)) : p.Skv;
    if (p.analytic && p.causal) key_end = (int)min((int64_t)key_end, max(p.q_pos_offset + p.Sq, (int64_t)1));
    const int q0 = pack ? 0 : qb * BM, qw0 = pack ? 16 * CB * (wave >> 2) : q0 + 16 * CB * wave;

    // visible keys: of the workgroup's rows (tiles to move), of the wavefront's rows (tiles to compute), of this
    // lane's two rows (element test).  row_bounds gives lane l the interval of row qw0 + l % 32.
    RowBounds rb = row_bounds(p, b, q0, pack ? 32 : BM, qw0, lane);
    if (nks > 1) {  // few query rows on a long cache: this workgroup takes one share of the keys
        const int c_lo = ksplit * p.pf_chunk, c_hi = c_lo + p.pf_chunk;
        rb.lo_wg = max(rb.lo_wg, c_lo), rb.hi_wg = min(rb.hi_wg, c_hi);
        rb.lo_w = max(rb.lo_w, c_lo), rb.hi_w = min(rb.hi_w, c_hi);
        rb.full_lo_w = max(rb.full_lo_w, c_lo), rb.full_hi_w = min(rb.full_hi_w, c_hi);
        rb.klo = max(rb.klo, c_lo), rb.khi = min(rb.khi, c_hi);
    }
    int klo[CB], khi[CB], row[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        klo[cb] = __shfl(rb.klo, 16 * cb + j, 64);
        khi[cb] = __shfl(rb.khi, 16 * cb + j, 64);
        row[cb] = qw0 + 16 * cb + j;
    }
    // the same in every lane: kept in scalar registers, so that the branches on them are plain jumps
    const int lo_wg = __builtin_amdgcn_readfirstlane(rb.lo_wg), hi_wg = __builtin_amdgcn_readfirstlane(rb.hi_wg);
    // the keys every row of the wavefront sees
    const int full_lo_w = __builtin_amdgcn_readfirstlane(rb.full_lo_w), full_hi_w = __builtin_amdgcn_readfirstlane(rb.full_hi_w);

    const uint16_t *kbase = (const uint16_t *)p.k + b * p.ks[0] + g * p.ks[1];
    const uint16_t *vbase = (const uint16_t *)p.v + b * p.vs[0] + g * p.vs[1];
    const float scale2 = p.scale * PW_LOG2E;

    // ---- tile movement: global -> LDS directly, no staging registers ---------------------------------------------------
    // A direct load writes the 64 lanes' 16 bytes to 1 KB of consecutive LDS, wherever each lane reads from.  The K tile
    // (rows of 2 D bytes at pitch KP) and the V tile (pitch VP) are therefore filled 1 KB at a time: piece i of a tile
    // covers its bytes [1024 i, 1024 i + 1024), lane l of it the 16 bytes at 1024 i + 16 l, which belong to row
    // pos / pitch, byte pos % pitch of the row; lanes that fall into the padding between rows or behind the last row
    // (each tensor's region is a whole number of pieces) fetch from beyond the buffer, i.e. zeros.  The NIK + NIV pieces of a tile pair are dealt round robin to the wavefronts.  K and V are raw buffers of
    // (Skv - 1) rows + 2 D bytes: a row beyond the key axis reads as zero (its scores are masked by the rows' intervals,
    // which end at the key count), so no clamps and no 64-bit address arithmetic in the loop.
    constexpr int NJ = (NIK + NIV + PW_WAVES - 1) / PW_WAVES;  // pieces per wavefront and tile pair
    const int krow_bytes = (int)p.ks[2] * 2, vrow_bytes = (int)p.vs[2] * 2;
    auto descriptor = [&](const uint16_t *base, int row_bytes) __attribute__((always_inline)) {
        const uint64_t ptr = (uint64_t)base;
        return uint4_t{(uint32_t)ptr, (uint32_t)(ptr >> 32) & 0xffffu, (uint32_t)((key_end - 1) * row_bytes + hd * 2),
                       0x00020000u};
    };
    const uint4_t krs = descriptor(kbase, krow_bytes), vrs = descriptor(vbase, vrow_bytes);
    int piece_voff[NJ];   // this lane's byte offset from the tile's first key (beyond the buffer for a lane without data)
    int piece_lds[NJ];    // where the piece starts in a stage (the same in every lane)
#pragma unroll
    for (int jj = 0; jj < NJ; jj++) {
        // (a wavefront whose share of the list is one short repeats the list's last piece: the same bytes to the same
        // place, and every wavefront then has exactly NJ loads per tile in flight, which the wait below counts on)
        const int idx = min(wave + PW_WAVES * jj, NIK + NIV - 1);
        const bool is_k = idx < NIK;
        const int i = is_k ? idx : idx - NIK;
        const int pos = 1024 * i + 16 * lane;
        const int pitch = is_k ? KP : VP, bytes = is_k ? K_BYTES : V_BYTES;
        const int r = pos / pitch, cbyte = pos % pitch;
        const bool active = pos < bytes && cbyte < 2 * hd;  // (the dims that pad the head up to D read as zero)
        piece_voff[jj] = active ? r * (is_k ? krow_bytes : vrow_bytes) + cbyte : 0x7ffffff0;
        piece_lds[jj] = (is_k ? 0 : V_AT) + 1024 * i;
    }
    auto issue_tile = [&](int j0, int stage_base) __attribute__((always_inline)) {
        // (uniform values; pinned to scalar registers, which is what the instruction takes.  A tile that starts beyond the
        // key axis is never used: the offset is clamped so that it stays inside 32 bits.)
        const int key0 = min(j0, p.Skv);
        const int lbase = (int)(uint32_t)(uintptr_t)lds_base + stage_base;
#pragma unroll
        for (int jj = 0; jj < NJ; jj++) {
            const bool is_k = min(wave + PW_WAVES * jj, NIK + NIV - 1) < NIK;  // the same for the whole wavefront
            const uint4_t rs = is_k ? krs : vrs;
            const int soff = __builtin_amdgcn_readfirstlane(key0 * (is_k ? krow_bytes : vrow_bytes));
            const int m0 = __builtin_amdgcn_readfirstlane(lbase + piece_lds[jj]);
            // written as assembly on purpose: the compiler would otherwise make every later LDS read of this wavefront
            // wait for these loads, whose data is not due before the next barrier
            // (no branch around it for the lanes without data: every wavefront must have the same number of loads in
            // flight per tile, which the waits count on)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                             :
                             : "s"(m0), "v"(piece_voff[jj]), "s"(rs), "s"(soff)
                             : "memory", "m0");
        }
    };
    // all direct loads of this wavefront have landed but those of the `newer` most recent tiles (NJ loads each; lanes
    // without a piece are masked off, the instruction is still issued and counted)
    auto wait_tiles = [&](int newer) __attribute__((always_inline)) {
        static_assert(2 * NJ <= 63, "vmcnt");
        if (newer == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        else if (newer == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NJ) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NJ) : "memory");
    };

    const int j_begin = (lo_wg / PW_KEYS) * PW_KEYS;
    const int ntiles = hi_wg > j_begin ? (hi_wg - j_begin + PW_KEYS - 1) / PW_KEYS : 0;
    if (ntiles > 0) issue_tile(j_begin, 0);  // issued first so the Q fetch below overlaps them
    if (NSTAGE > 2 && ntiles > 1) issue_tile(j_begin + PW_KEYS, STAGE);

    // Q^T operand: column j of block cb, dims 32 kb + 8 q4 .. +8 (rows beyond Sq repeat the last row; never stored)
    vec8 qreg[CB][KB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        const uint16_t *qp = (const uint16_t *)p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)min(row[cb], p.Sq - 1) * p.qs[2];
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
            uint4_t raw = {0, 0, 0, 0};
            if (32 * kb + 8 * q4 < hd) raw = *(const uint4_t *)(qp + 32 * kb + 8 * q4);
            qreg[cb][kb] = __builtin_bit_cast(vec8, raw);
        }
    }

    float4_t o[CB][NB];
    float m[CB], l[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) o[cb][nb] = float4_t{0.f, 0.f, 0.f, 0.f};
        m[cb] = -INFINITY, l[cb] = 0.0f;
    }

    // A tile in three parts.  tile_front brings tile t into LDS and computes the wavefront's masked scores (log2 units)
    // and their per-column maxima; move_reference raises the reference maximum of the columns that need it and
    // rescales O and l; tile_back turns the scores into probabilities and adds P . V.  The reference maximum of a
    // column moves only when a tile exceeds it by more than 2^8 (probabilities then reach 2^8 at most, well inside
    // f16 / bf16 range), which after the first tile almost never happens: the loop below runs front + back and leaves
    // for move_reference only then, so that in the loop nothing but the matrix instructions touches O.
    float sv[CB][8], mx[CB];
    int sbase = 0;
    // (A tile none of the wavefront's rows sees is not skipped: its scores are -inf, its probabilities 0.  A jump
    // around the P . V block makes the compiler carry two copies of O and move one into the other on every tile,
    // which costs more than the few such tiles on the diagonal of a causal mask.)
    auto tile_front = [&](int t) __attribute__((always_inline)) -> bool {  // true: move the reference first
        const int j0 = j_begin + t * PW_KEYS;
        sbase = (t % NSTAGE) * STAGE;
        // tile t has landed: all of this wavefront's loads but those of the tiles issued after it
        wait_tiles(min(ntiles - 1 - t, NSTAGE - 2));
        __syncthreads();  // tile t is in LDS; every wavefront is done with tile t - 1, whose stage the next issue takes
        if (t + NSTAGE - 1 < ntiles) issue_tile(j0 + (NSTAGE - 1) * PW_KEYS, ((t + NSTAGE - 1) % NSTAGE) * STAGE);
        const bool all_visible = j0 >= full_lo_w && j0 + PW_KEYS <= full_hi_w;  // no element test needed

        // S^T[key][col] = K . Q^T : two 16-key halves, every K operand read serves both column blocks
        // (contraction blocks outermost: four accumulators take turns, so that a matrix instruction never waits for
        // the result of the one just issued)
        float4_t s[CB][2];
#pragma unroll
        for (int hf = 0; hf < 2; hf++)
#pragma unroll
            for (int cb = 0; cb < CB; cb++) s[cb][hf] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
#pragma unroll
            for (int hf = 0; hf < 2; hf++) {
                const uint4_t raw = *PWLDS_PTR(uint4_t, sbase + (16 * hf + j) * KP + (32 * kb + 8 * q4) * 2);
#pragma unroll
                for (int cb = 0; cb < CB; cb++)
                    s[cb][hf] = WideMma<T>::mfma(__builtin_bit_cast(vec8, raw), qreg[cb][kb], s[cb][hf]);
            }
        }
        bool grow = false;
#pragma unroll
        for (int cb = 0; cb < CB; cb++) {
            // element (hf, r) is key j0 + 16 hf + 4 q4 + r for column j of block cb
            if (all_visible) {
#pragma unroll
                for (int e = 0; e < 8; e++) sv[cb][e] = s[cb][e >> 2][e & 3] * scale2;
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int key = j0 + 16 * (e >> 2) + 4 * q4 + (e & 3);
                    sv[cb][e] = (key >= klo[cb] && key < khi[cb]) ? s[cb][e >> 2][e & 3] * scale2 : -INFINITY;
                }
            }
            float x = sv[cb][0];
#pragma unroll
            for (int e = 1; e < 8; e++) x = fmaxf(x, sv[cb][e]);
            mx[cb] = pw_quad_max(x);
            grow |= (m[cb] == -INFINITY) ? (mx[cb] > -INFINITY) : (mx[cb] > m[cb] + PW_RESCALE_SLACK);
        }
        return __builtin_amdgcn_ballot_w64(grow) != 0;
    };
    auto move_reference = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int cb = 0; cb < CB; cb++) {
            const bool first = m[cb] == -INFINITY;
            const bool grow = first ? (mx[cb] > -INFINITY) : (mx[cb] > m[cb] + PW_RESCALE_SLACK);
            const float m_new = grow ? mx[cb] : m[cb];
            const float corr = (grow && !first) ? __builtin_amdgcn_exp2f(m[cb] - m_new) : 1.0f;
            m[cb] = m_new;
            l[cb] *= corr;
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
                for (int r = 0; r < 4; r++) o[cb][nb][r] *= corr;
        }
    };
    auto tile_back = [&]() __attribute__((always_inline)) {
        vec8 pop[CB];
#pragma unroll
        for (int cb = 0; cb < CB; cb++) {
            const float m_safe = (m[cb] == -INFINITY) ? 0.0f : m[cb];
            float pe[8], psum = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                pe[e] = __builtin_amdgcn_exp2f(sv[cb][e] - m_safe);
                psum += pe[e];
            }
            l[cb] += psum;
            // P^T operand: contraction slot (q4, e) is key 4 q4 + e (e < 4) or 16 + 4 q4 + e - 4
            const uint4_t praw = {WideMma<T>::pack2(pe[0], pe[1]), WideMma<T>::pack2(pe[2], pe[3]),
                                  WideMma<T>::pack2(pe[4], pe[5]), WideMma<T>::pack2(pe[6], pe[7])};
            pop[cb] = __builtin_bit_cast(vec8, praw);
        }
        // O^T[dim][col] += V^T . P^T: the transposing load hands lane i of a 16-lane block V[row0 + 0..3][dim0 + i];
        // the lane supplies the address of row0 + i / 4, dims dim0 + 4 (i % 4)
        const int trow = 4 * q4 + (j >> 2);
        const int tcol = 4 * (j & 3) * 2;
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const short4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                PWLDS_PTR(short4_t, sbase + V_AT + trow * VP + nb * 32 + tcol));
            const short4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                PWLDS_PTR(short4_t, sbase + V_AT + (16 + trow) * VP + nb * 32 + tcol));
            const uint2w_t u0 = __builtin_bit_cast(uint2w_t, a0), u1 = __builtin_bit_cast(uint2w_t, a1);
            const uint4_t araw = {u0[0], u0[1], u1[0], u1[1]};
#pragma unroll
            for (int cb = 0; cb < CB; cb++)
                o[cb][nb] = WideMma<T>::mfma(__builtin_bit_cast(vec8, araw), pop[cb], o[cb][nb]);
        }
    };
    for (int t = 0;;) {
        for (; t < ntiles; t++) {
            if (tile_front(t)) break;
            tile_back();
        }
        if (t >= ntiles) break;
        move_reference();
        tile_back();
        t++;
    }

    // ---- epilogue: out[row][16 nb + 4 q4 + r] = O^T / l (no visible key: 0 / 0 = NaN like the reference) -------
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        const float l_col = pw_quad_sum(l[cb]);
        if (row[cb] >= p.Sq) continue;
        if (nks > 1) {
            // this share's state: O unnormalised, then (m, l); the merge kernel normalises
            float *ws = p.partials + ((((int64_t)b * p.H + h) * p.Sq + row[cb]) * nks + ksplit) * p.pf_pitch;
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
                if (16 * nb + 4 * q4 < hd) *(float4_t *)(ws + 16 * nb + 4 * q4) = o[cb][nb];
            if (q4 == 0) {
                ws[hd] = m[cb];
                ws[hd + 1] = l_col;
            }
            continue;
        }
        const int64_t ob = b * p.os[0] + h * p.os[1] + (int64_t)row[cb] * p.os[2];
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float val = o[cb][nb][r] / l_col;
                const int64_t oi = ob + (int64_t)(16 * nb + 4 * q4 + r) * p.os[3];
                if (16 * nb + 4 * q4 >= hd) continue;
                if (p.out_f32) ((float *)p.out)[oi] = val;
                else ((T *)p.out)[oi] = from_float<T>(val);
            }
    }
}

// Wavefronts per workgroup: eight wavefronts of 16 rows (two per SIMD, half the register file each), which hide each
// other's dependent phases but read every K and V operand from LDS for half as many matrix instructions as four
// wavefronts of 32 rows would.  Measured (f16, 4096 x 4096 causal) while the tiles still went through staging registers:
// +15 % at head_dim 160, +16 % at 192, +6 % at 224 and -5 % at 256 (249 of 256 registers); with the tiles loaded
// straight into LDS (218 registers at 256) eight are ahead there too, 535 against 501 TFLOP/s.  The four-wavefront
// form <4, 2> is kept in the template for such measurements.
constexpr int wide_waves(int) { return 8; }

template <typename T, int D>
void launch_wide_d(const AttnParams &p, int bm, const dim3 &grid, int nqb, hipStream_t stream) {
    if (bm == 64) {
        FHIP_LAUNCH_MAIN((prefill_mfma_wide_kernel<T, D, 4, 1>), grid, dim3(256), stream, p, p, nqb);
    } else if (bm == 256) {
        if constexpr (D <= 192) FHIP_LAUNCH_MAIN((prefill_mfma_wide_kernel<T, D, 8, 2>), grid, dim3(512), stream, p, p, nqb);
    } else {
        constexpr int W = wide_waves(D);
        FHIP_LAUNCH_MAIN((prefill_mfma_wide_kernel<T, D, W, 8 / W>), grid, dim3(64 * W), stream, p, p, nqb);
    }
}

template <typename T>
int launch_wide_t(const AttnParams &p_in, hipStream_t stream) {
    AttnParams p = p_in;
    p.pf_pack = prefill_mfma_pack(p.B, p.H, p.G, p.Sq, p.Skv, p.cus > 0 ? p.cus : 256);
    // A grid of fewer than two 128-row workgroups per CU that cannot split the keys (a causal prompt of up to a few
    // thousand tokens) runs as 64-row workgroups, two per CU: twice the workgroups of half the length, which fill idle
    // CUs and even out the long and short row blocks of a causal mask, each reading K and V from LDS for half as
    // many matrix instructions (f16, head_dim 256, 16 heads: 512 tokens 48 -> 33 us, 1024: 72 -> 52, 2048: 125 -> 108,
    // 3072: 179 -> 170).
    // Above head_dim 192 every call but the split and packed ones of up to 64 query rows runs on the kernel of four
    // 32-row wavefronts (attn_prefill_mfma_rows32.hip), whatever the grid: f16, head_dim 256, causal, 8 heads: 512 tokens
    // 27.9 -> 24.5 us, 1024: 44.0 -> 36.1, 2048: 77.8 -> 60.3, 4096: 172 -> 116; 16 heads, 4096: 207 -> 152.
    if (prefill_mfma_rows32_takes(p))
        return launch_prefill_mfma_rows32(p, std::is_same<T, half_t>::value ? FHIP_F16 : FHIP_BF16, stream);
    const long wgs128 = (long)p.B * p.H * ((p.Sq + PW_BM - 1) / PW_BM);
    // (With the keys split, up to 64 rows are one row block either way: the 64-row form computes half as much per tile
    // and runs two workgroups per CU: f16, head_dim 256, B8 x 16 heads, 64 rows on 8192 keys 271 -> 181 us.)
    const bool small = p.pf_nsplit <= 1 ? wgs128 < 2 * p.cus : p.Sq <= 64;
    int bm = (!p.pf_pack && small) ? 64 : PW_BM;
    // Up to head_dim 192 a wavefront can hold 32 rows (two column blocks: every K and V operand read from LDS then feeds
    // two matrix instructions): 256-row workgroups where those still give every CU one (f16, 4096 x 4096 causal:
    // head_dim 160 497 -> 559 TFLOP/s, 192 450 -> 511; at 224 and 256 the registers do not suffice)
    const long wgs256 = (long)p.B * p.H * ((p.Sq + 255) / 256);
    const bool big = wgs256 >= p.cus;
    if (!p.pf_pack && !small && p.pf_nsplit <= 1 && p.D <= 192 && big) bm = 256;
    const int nqb = p.pf_pack ? 1 : (p.Sq + bm - 1) / bm;
    const long blocks = (long)nqb * p.B * (p.pf_pack ? p.H / 4 : p.H) * (p.pf_nsplit > 1 ? p.pf_nsplit : 1);
    if (blocks > 0x7fffffffL) {
        set_error("prefill: too many workgroups (%ld)", blocks);
        return FHIP_ERR_UNSUPPORTED;
    }
    const dim3 grid((unsigned)blocks);
    if (p.D % 8 != 0 || p.D < 8 || p.D > 256) {
        set_error("wide prefill MFMA kernel: head_dim %d is not a multiple of 8 up to 256", p.D);
        return FHIP_ERR_UNSUPPORTED;
    }
    switch ((p.D + 31) / 32 * 32) {  // the kernel's D is head_dim rounded up to a multiple of 32
        case 32: launch_wide_d<T, 32>(p, bm, grid, nqb, stream); break;
        case 64: launch_wide_d<T, 64>(p, bm, grid, nqb, stream); break;
        case 96: launch_wide_d<T, 96>(p, bm, grid, nqb, stream); break;
        case 128: launch_wide_d<T, 128>(p, bm, grid, nqb, stream); break;
        case 160: launch_wide_d<T, 160>(p, bm, grid, nqb, stream); break;
        case 192: launch_wide_d<T, 192>(p, bm, grid, nqb, stream); break;
        case 224: launch_wide_d<T, 224>(p, bm, grid, nqb, stream); break;
        default: launch_wide_d<T, 256>(p, bm, grid, nqb, stream); break;
    }
    FHIP_HIP_CHECK(hipGetLastError());
    if (p.pf_nsplit > 1) return launch_prefill_merge(p, std::is_same<T, half_t>::value ? FHIP_F16 : FHIP_BF16, stream);
    return FHIP_OK;
}

}  // namespace

// Few query rows on a long cache: 128-row query blocks alone leave most CUs idle, so the keys are split over workgroups
// too, down to 1024 keys per share, until there are about two workgroups per CU (the rule of the other tiled kernels).
void prefill_mfma_wide_plan(int B, int H, int G, int Sq, int Skv, bool causal_square, int compute_units, int *nsplit, int *chunk) {
    *nsplit = 1;
    *chunk = Skv;
    if (causal_square) return;
    const int pack = prefill_mfma_pack(B, H, G, Sq, Skv, compute_units);
    const long wgs = (long)B * (pack ? H / 4 : H) * ((Sq + PW_BM - 1) / PW_BM);
    // places for workgroups: one per CU, two for the 64-row form that serves up to 64 rows.  A tile takes this kernel
    // microseconds whatever part of the row block is real, so a grid that leaves places empty splits its keys.
    const long places = (!pack && Sq <= 64 ? 2L : 1L) * compute_units;
    if (wgs >= places) return;
    // The share count that needs the fewest tile steps: rounds of `places` workgroups, each walking its share of the
    // keys tile by tile, plus a few steps for parking and merging the partial results of a split.
    const long most = Skv / 1024 < 64 ? Skv / 1024 : 64;
    long best_ns = 1, best_cost = (Skv + PW_KEYS - 1) / PW_KEYS;
    for (long ns = 2; ns <= most; ns++) {
        const long rounds = (wgs * ns + places - 1) / places;
        const long tiles = ((Skv + ns - 1) / ns + PW_KEYS - 1) / PW_KEYS;
        const long cost = rounds * tiles + 4;
        if (cost < best_cost) best_cost = cost, best_ns = ns;
    }
    if (best_ns < 2) return;
    long c = (Skv + best_ns - 1) / best_ns;
    c = (c + PW_KEYS - 1) / PW_KEYS * PW_KEYS;
    *chunk = (int)c;
    *nsplit = (int)((Skv + c - 1) / c);
}

int launch_prefill_mfma_wide(const AttnParams &p, fhip_dtype dtype, hipStream_t stream) {
    if (dtype == FHIP_F16) return launch_wide_t<half_t>(p, stream);
    if (dtype == FHIP_BF16) return launch_wide_t<bf16_t>(p, stream);
    set_error("wide prefill MFMA kernel takes f16/bf16 only");
    return FHIP_ERR_UNSUPPORTED;
}

}  // namespace fhip
