// How the prefill launch maps workgroup ids to (head, query tile): plain C++ shared by the kernel, the launcher and
// the CPU test of the mapping (which checks that every pair is visited exactly once for any launch shape).
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define TSATTN_HD __host__ __device__
#else
#define TSATTN_HD
#endif

namespace tsattn {

// A launch-constant divisor with its reciprocal: x / d is one multiply-high and a correction by at most one.
// Valid for x < 2^31.
struct WgDiv {
    uint32_t d, m;
};

inline WgDiv wg_make_div(uint32_t d)
{
    WgDiv r;
    r.d = d ? d : 1;
    // ceil(2^32 / d) overestimates the quotient by at most one; it does not fit 32 bits for d = 1, where
    // 2^32 - 1 underestimates by exactly one instead
    r.m = r.d == 1 ? 0xffffffffu : (uint32_t)(((1ull << 32) + r.d - 1) / r.d);
    return r;
}

TSATTN_HD inline uint32_t wg_divmod(uint32_t x, WgDiv by, uint32_t &rem)
{
    uint32_t q = (uint32_t)(((uint64_t)x * by.m) >> 32);
    int32_t r = (int32_t)(x - q * by.d);
    if (r < 0) { --q; r += (int32_t)by.d; }
    if (r >= (int32_t)by.d) { ++q; r -= (int32_t)by.d; }
    rem = (uint32_t)r;
    return q;
}

struct WgMap {
    int period_tiles;  // T: query tiles per period of equal span structure, 0 = unknown
    int period_group;  // G: units per group of the period-aware order, 0 = that order is not used
    int units_per_xcd; // R: (head group, sequence) units per XCD
    int hg_shift;      // log2 of the heads that share a cache line (d = 64 with an even head count: 1)
    WgDiv by_qtiles, by_group_wgs, by_group_units, by_seqs;
};

// Plans the mapping of a launch of n_qtiles * n_heads workgroups.  The period-aware order is usable only if every
// XCD's share of the grid is a whole number of (head group, sequence) units; units are then walked in groups whose
// K and V rows (kv_bytes_per_value * period * d bytes per head: 2 for 8-bit K and V) stay within about the size of the XCD's 4 MB L2 (the rows are
// streamed, so slightly more than it still pays).
inline WgMap wg_plan(int n_qtiles, int n_heads, int head_dim, int rows_per_tile, int period_tiles, int kv_bytes_per_value = 2)
{
    WgMap m;
    m.period_tiles = period_tiles;
    m.period_group = 0;
    m.units_per_xcd = 0;
    const int hg = (head_dim == 64 && (n_heads & 1) == 0) ? 2 : 1;
    m.hg_shift = hg == 2 ? 1 : 0;
    m.by_qtiles = wg_make_div((uint32_t)n_qtiles);
    m.by_group_wgs = m.by_group_units = m.by_seqs = wg_make_div(1);
    const int T = period_tiles;
    const int64_t n_wg = (int64_t)n_qtiles * n_heads, per_xcd = n_wg / 8;
    if (T > 1 && n_wg % 8 == 0 && per_xcd % (T * hg) == 0 && n_qtiles % T == 0) {
        const int R = (int)(per_xcd / (T * hg));
        const int64_t unit_bytes = (int64_t)kv_bytes_per_value * T * rows_per_tile * head_dim * hg;
        int G = 1;
        for (int c = 1; c <= R; ++c)
            if (R % c == 0 && c * unit_bytes <= (5 << 20)) G = c;
        m.period_group = G;
        m.units_per_xcd = R;
        m.by_group_wgs = wg_make_div((uint32_t)(G * T * hg));
        m.by_group_units = wg_make_div((uint32_t)(G * hg));
        m.by_seqs = wg_make_div((uint32_t)(n_qtiles / T));
    }
    return m;
}

// (head, query tile) of workgroup `block` of a launch of n_wg = n_qtiles * n_heads workgroups.
//
// Workgroups are handed to the 8 XCDs round-robin; each XCD gets a contiguous run of (head, query tile) pairs:
// equal work per XCD, and the K/V rows a run shares stay in its L2.  With d = 64 one 128-byte line of K or V holds
// the rows of two heads: consecutive workgroups then alternate between the two heads of a pair on the same query
// tile, so the pair shares the line in L2.
TSATTN_HD inline void wg_locate(const WgMap &m, uint32_t block, uint32_t n_wg, int n_qtiles, int &head, int &tile)
{
    const int hs = m.hg_shift, hg = 1 << hs;
    if (m.period_group > 0) {
        // The caller has said that the batch repeats the same span structure every T query tiles (equal-length
        // sequences, causal): each XCD still gets a contiguous run of (head group, sequence) units, but walks groups
        // of G units position by position from the end of the sequences to their start: the longest rows of every
        // unit first, the shortest last, so the launch does not end on a few long-running workgroups.
        const int T = m.period_tiles, G = m.period_group;
        const uint32_t x = block & 7, i = block >> 3; // XCD and index inside its run
        uint32_t j, rem, seq;
        const uint32_t grp = wg_divmod(i, m.by_group_wgs, j);          // / (G * T * hg)
        const uint32_t pos_rank = wg_divmod(j, m.by_group_units, rem); // / (G * hg)
        const uint32_t U = x * (uint32_t)m.units_per_xcd + grp * (uint32_t)G + (rem >> hs);
        const uint32_t hgrp = wg_divmod(U, m.by_seqs, seq);            // / (n_qtiles / T)
        head = (int)((hgrp << hs) + (rem & (uint32_t)(hg - 1)));
        tile = (int)(seq * (uint32_t)T + ((uint32_t)T - 1 - pos_rank));
    } else {
        uint32_t wg = block, t;
        if ((n_wg & 7) == 0) wg = (block & 7) * (n_wg >> 3) + (block >> 3);
        const uint32_t hgrp = wg_divmod(wg >> hs, m.by_qtiles, t);
        head = (int)((hgrp << hs) + (wg & (uint32_t)(hg - 1)));
        tile = n_qtiles - 1 - (int)t; // long rows first
    }
}

} // namespace tsattn
