// Arguments of the decode / verify-window launches, as the launchers resolve them from the C ABI's parameters.
#pragma once
#include <type_traits>

#include "pkv_common.hpp"

namespace pkv {

constexpr int kMaxListedBlocks = 1024;      // block ids a token's list may hold (they are copied to LDS)
// A split launch lists every row's last partition (usually a partial piece, the smallest unit of work) after all other
// partitions, in this many classes of decreasing size, so that the units that start last are the smallest.
constexpr int kTailClasses = 4;

struct AttendArgs {
    const uint8_t* q;
    const uint8_t* kp;
    const uint8_t* vp;
    const float* ks;
    const float* vs;
    const float* hm;
    const int32_t* tables;
    const int32_t* rows;      // entry r at rows[r * rows_step]: int32 entries (step 1) or the low words of int64 ones (step 2)
    int rows_step;
    const int32_t* starts;
    const int32_t* counts;
    const int64_t* firsts;
    const int32_t* offsets;
    float* po;
    float* pm;
    float* pl;
    void* out;
    float* lse;
    const float* sinks;
    const int32_t* parents;      // draft trees: each token's parent column, int32 ...
    const int64_t* parents64;    // ... or int64; both null: plain causal windows
    const int32_t* blocks;       // block-sparse lists [tokens][blocks_k], or null: every position
    unsigned* ticket;      // two zeroed counters of the unit-pulling launches: next unit, workgroups done
    int64_t q_st, q_sh, o_st, o_sh, tab_stride, blocks_stride;
    int dk, dv;      // key and value head widths
    int fast128;     // keys and values 128 wide: the bandwidth kernel where the pages (or block lists) allow it
    int tab_width, n_rows, columns, hq, hkv, g, page, page_shift, parts, piece, sliding, out_dtype, tiles, max_keys, heads_per_wave, units_x, units_y, query_tiles;
    int blocks_k, block_size, listed_keys;      // listed_keys = blocks_k * block_size: the positions a list's run holds
    Div32 block_div;
    float sscale, k_mult, v_mult;
    // Fresh rows (attend's fresh=): row r reads its positions from f_firsts[r * f_per_row] on from rows
    // position - f_shifts[r * f_per_row] of fk / fv ([f_rows][kv_heads][dim], q's 16-bit type, unscaled) instead of the
    // pages. fk null: every position from the pages.
    const uint8_t* fk;
    const uint8_t* fv;
    const int64_t* f_shifts;
    const int64_t* f_firsts;
    int64_t f_stride_k, f_stride_v, f_rows;
    int f_per_row;
    // Derived keys: the inverse frequencies [derive_rot / 2], then the norm's weight [dk] when derive_weighted; null:
    // keys from their pages.
    const float* derive_table;
    float derive_eps;
    int derive_rot, derive_weighted;
    int narrow;   // 64-wide heads read in pairs as 128-wide ones: hkv, g, dk and dv above are the pairs' (half, twice, 128, 128)
    int iqk;      // INT8 pages: the queries as INT8 codes at each row's own scale (prefill's int8_qk read as windows)
};

// A workgroup barrier that orders the shared arrays only: a wavefront waits for its own LDS traffic, then for the
// others. __syncthreads() would also wait until the wavefront's global stores (a unit's partials, which only the next
// kernel reads) have drained, a memory round trip at every barrier of a unit's end.
PKV_DEV void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// A 16-byte (or 8-byte) load of value rows, which are read once: nontemporal, so the caches do not keep them (measured
// +4 % on the decode launch; the same hint on the key rows measured -1 %, so those stay plain loads).
PKV_DEV uint4 load_once16(const uint8_t* p) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
PKV_DEV uint2 load_once8(const uint8_t* p) {
    const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    return make_uint2(v.x, v.y);
}

// Draft trees: the set of window columns column `c` of the row whose first token is `start` sees (its ancestors and
// itself) as a 64-bit mask, by walking the parent links (parents come before children, so at most c links; a link that
// does not point at an earlier column ends the walk).
PKV_DEV unsigned long long ancestors(const AttendArgs& a, int start, int c) {
    unsigned long long set = 1ull << c;
    int at = c;
    for (int hop = 0; hop < 64 && at > 0; ++hop) {
        const int64_t par = a.parents ? (int64_t)a.parents[start + at] : a.parents64[start + at];
        if (par < 0 || par >= at) break;
        at = (int)par;
        set |= 1ull << at;
    }
    return set;
}

}   // namespace pkv
