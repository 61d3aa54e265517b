// Visible key ranges of the query rows a prefill workgroup / wavefront / lane owns.
//
// Every supported mask leaves each query row ONE interval [klo, khi) of visible keys:
//   - analytic description: j <= r + off (causal), j + window > r + off (sliding window)
//   - per-batch key range: kv_lens[b], or the interval form of a BatchKeyMask
//   - per-row interval form of a QKMask (mask_intervals.hip)
// The tiled kernels need the row's own interval (element test), the union over a wavefront's and a
// workgroup's rows (which tiles to visit / load) and the intersection over a wavefront's rows (tiles
// that need no element test).
#pragma once
#include "common.h"
#include "device_utils.h"

namespace fhip {

struct RowBounds {
    int lo_wg, hi_wg;          // union over the workgroup's rows
    int lo_w, hi_w;            // union over this wavefront's 32 rows
    int full_lo_w, full_hi_w;  // intersection over this wavefront's rows
    int klo, khi;              // this lane's row
};

// q0: first row of the workgroup, bm: rows per workgroup, qw0: first row of the wavefront (32 rows,
// lane ln = lane % 32 owns row qw0 + ln).  iv: the interval form of the mask tensor, or NULL.
__device__ __forceinline__ RowBounds row_bounds(const AttnParams &p, const int2 *iv, int b, int q0, int bm, int qw0, int lane) {
    const int ln = lane & 31;
    int kv_lo = 0, kv_hi = p.Skv;
    if (p.kv_lens) kv_hi = min(kv_hi, max(p.kv_lens[b], 0));
    if (iv && p.mask_kind == FHIP_MASK_BATCH_KEY) {
        const int2 t = iv[b];
        kv_lo = max(kv_lo, t.x);
        kv_hi = min(kv_hi, t.y);
    }
    RowBounds r;
    if (!(iv && p.mask_kind == FHIP_MASK_QK)) {
        const int64_t off = p.q_pos_offset;
        auto row_lo = [&](int q) __attribute__((always_inline)) -> int {
            return (p.analytic && p.window > 0) ? (int)max((int64_t)kv_lo, (int64_t)q + off - p.window + 1) : kv_lo;
        };
        auto row_hi = [&](int q) __attribute__((always_inline)) -> int {
            return (p.analytic && p.causal) ? (int)min((int64_t)kv_hi, (int64_t)q + off + 1) : kv_hi;
        };
        // both ends move forward with the row index
        const int q_last_wg = min(q0 + bm - 1, p.Sq - 1);
        const int q_last_w = min(qw0 + 31, p.Sq - 1);
        const int q_first_w = min(qw0, p.Sq - 1);
        const int qrow = min(qw0 + ln, p.Sq - 1);
        r.lo_wg = row_lo(q0), r.hi_wg = row_hi(q_last_wg);
        r.lo_w = row_lo(q_first_w), r.hi_w = row_hi(q_last_w);
        r.full_lo_w = row_lo(q_last_w), r.full_hi_w = row_hi(q_first_w);
        r.klo = row_lo(qrow), r.khi = row_hi(qrow);
        return r;
    }
    constexpr int NONE = 0x7fffffff;
    auto load_row = [&](int q, int &lo, int &hi) __attribute__((always_inline)) {
        const int2 t = iv[min(q, p.Sq - 1)];
        lo = max(kv_lo, t.x);
        hi = min(kv_hi, t.y);
        if (hi <= lo) lo = hi = 0;  // nothing visible
    };
    auto wave_min = [&](int x) __attribute__((always_inline)) -> int {
        return __builtin_amdgcn_readfirstlane(wave_reduce_i(x, [](int a, int b) { return min(a, b); }));
    };
    auto wave_max = [&](int x) __attribute__((always_inline)) -> int {
        return __builtin_amdgcn_readfirstlane(wave_reduce_i(x, [](int a, int b) { return max(a, b); }));
    };
    load_row(qw0 + ln, r.klo, r.khi);
    const bool empty = r.khi == 0;
    r.lo_w = wave_min(empty ? NONE : r.klo);
    r.hi_w = wave_max(r.khi);
    r.full_lo_w = wave_max(empty ? NONE : r.klo);  // one empty row: no tile is fully visible
    r.full_hi_w = wave_min(r.khi);
    if (r.hi_w <= r.lo_w) r.lo_w = r.hi_w = 0;
    int lo_u = NONE, hi_u = 0;
    for (int q = q0 + lane; q < q0 + bm; q += 64) {
        int lo, hi;
        load_row(q, lo, hi);
        if (hi > 0) lo_u = min(lo_u, lo);
        hi_u = max(hi_u, hi);
    }
    r.lo_wg = wave_min(lo_u);
    r.hi_wg = wave_max(hi_u);
    if (r.hi_wg <= r.lo_wg) r.lo_wg = r.hi_wg = 0;
    return r;
}

__device__ __forceinline__ RowBounds row_bounds(const AttnParams &p, int b, int q0, int bm, int qw0, int lane) {
    return row_bounds(p, p.iv, b, q0, bm, qw0, lane);
}

}  // namespace fhip
