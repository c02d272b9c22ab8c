// Paged decode / verify-window attention for 128-wide heads over pages of a multiple of 16 positions: the bandwidth
// path of the split and fused launches.
//
// The kernel is bound by HBM reads of K and V; everything else is arranged so that nothing but those reads limits it.
// The two products of a step run on the matrix pipe, which a decode kernel otherwise leaves idle, because the vector
// pipe cannot keep up with 8-bit pages at HBM rate (one v_dot2 per two multiply-adds, plus the conversions, was two
// thirds of its cycles): a step is 16 positions of one KV head,
//   S^T[16 positions][16 query rows] = K[16][128] . Q^T      4 x v_mfma_f32_16x16x32 (bf16 / f16 operands)
//   O^T[128 dims][16 query rows]    += V^T[128][16] . P^T    8 x v_mfma_f32_16x16x16
// with operands laid out so that nothing is shuffled between memory and the matrix pipe:
//   keys    lane (p = lane % 16, u = lane / 16) loads 16-byte pieces of the row of position p; piece c holds dims
//           32 c + 8 u .. + 7, the eight contraction elements the first product's A operand wants from that lane
//           (8-bit pages: two loads of 16 codes, converted to 16-bit pairs, exactly);
//   values  lane (i = lane % 16, u) loads 16 bytes (dims 8 i .. 8 i + 7) of the rows of positions 4 u .. 4 u + 3: a
//           load instruction fetches four whole rows. The second product's A operand for dims {8 i + j} is the four
//           positions' element j as two 16-bit pairs: one v_perm_b32 each;
//   scores  come out with lane (c = lane % 16, u) holding query row c at positions 4 u .. 4 u + 3, which is exactly
//           the B operand layout of the second product: the probabilities go from the softmax to the matrix pipe
//           as two packed registers, no LDS, no shuffle.
// The 16 query rows of a tile are rows of the flattened (column, group head) list, so the GQA group's heads share
// every K/V byte read once. A wavefront serves HW adjacent KV heads (2 where the head count is even) in ONE matrix tile:
// a step is then 8 positions of both heads (rows 0 .. 7 of the tile the first head's positions, rows 8 .. 15 the
// second's, columns 0 .. 7 the first head's query rows, 8 .. 15 the second's; the products of one head's keys with the
// other head's queries are masked), so a load instruction fetches both heads' rows of a position, 512 contiguous bytes
// of 16-bit pages: what the HBM system streams best from randomly placed pages.
// Softmax state: the running maximum of a query row is kept equal in the four lanes that hold the row (two
// v_permlane swaps a step), the sums per lane until the unit's end. NT tiles are in flight per wavefront; every load
// of the loop is unconditional, so the waits are exact counts.
//
// Row-exactness: position n is always read in the same step of the same wavefront of its unit, at the same place of
// the matrix operands; the matrix pipe computes each output element from its own row and column only; every other
// reduction is a fixed tree. So a column's bits depend on its own query and keys, `piece`, `partitions`, the page kind
// and the cache geometry only: not on the rows beside it, the launch's width, the tile it falls in, which workgroup
// served it, or `fused`.
#pragma once
#include "pkv_attend_args.hpp"

namespace pkv {

template <bool F16>
PKV_DEV f32x4 mfma_k32(u32x4 a, u32x4 b, f32x4 c) {
    if constexpr (F16) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
}
template <bool F16>
PKV_DEV f32x4 mfma_k16(u32x2 a, u32x2 b, f32x4 c) {
    typedef __attribute__((ext_vector_type(4))) short s16x4;
    typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
    if constexpr (F16) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
    }
}

template <bool F16>
PKV_DEV uint32_t pair16(float a, float b) {      // two FP32 values as one 16-bit pair, round to nearest even
    if constexpr (F16) return pack_f16(a, b);
    typedef __attribute__((ext_vector_type(2))) __bf16 pair_t;
    const pair_t r = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(uint32_t, r);
}

// Four codes of one word as two packed 16-bit pairs (x: codes 0,1; y: codes 2,3), exactly.
template <int KIND>
PKV_DEV u32x2 codes4_to_pairs(uint32_t w) {
    if constexpr (KIND == 3) {
        const float f0 = (float)(int8_t)w, f1 = (float)(int8_t)(w >> 8), f2 = (float)(int8_t)(w >> 16), f3 = (float)(int8_t)(w >> 24);
        return u32x2{__builtin_amdgcn_perm(f2u(f1), f2u(f0), 0x07060302), __builtin_amdgcn_perm(f2u(f3), f2u(f2), 0x07060302)};
    } else {
        return u32x2{__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)w, 1.0f, false)),
                     __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)w, 1.0f, true))};
    }
}

// The maximum (sum) of x over the four lanes 16 apart that hold one tile column: two v_permlane swaps.
PKV_DEV float max_across_quarters(float x) {
    const int v = (int)f2u(x);
    auto a = __builtin_amdgcn_permlane16_swap(v, v, false, false);      // rows (0,1) and (2,3) meet
    const float y = __builtin_fmaxf(u2f((uint32_t)a[0]), u2f((uint32_t)a[1]));
    const int w = (int)f2u(y);
    auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);      // halves meet
    return __builtin_fmaxf(u2f((uint32_t)b[0]), u2f((uint32_t)b[1]));
}
PKV_DEV float sum_across_quarters(float x) {      // (row 0 + row 1) + (row 2 + row 3), the same bits in all four lanes
    const int v = (int)f2u(x);
    auto a = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    const float y = u2f((uint32_t)a[0]) + u2f((uint32_t)a[1]);
    const int w = (int)f2u(y);
    auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return u2f((uint32_t)b[0]) + u2f((uint32_t)b[1]);
}

template <int KIND, int DH>
struct Tile {
    using VVec = typename std::conditional<KIND == 0, u32x4, u32x2>::type;
    u32x4 k[(KIND == 0 ? 4 : 2) * DH];      // the lane's pieces of its position's K row
    VVec v[4][DH];                           // the lane's 8 dims (of each 128-wide half) of the V rows of its quarter's four positions
    float ks[KIND >= 2 ? 4 : 1], vs[KIND >= 2 ? 4 : 1];      // row-scaled kinds: the scales of positions 4 u .. 4 u + 3
};

constexpr int kTileRows = 16;      // query rows (columns of S^T) a tile holds
constexpr int kLdsRows = 512;      // batch rows whose descriptors a workgroup keeps in LDS (the others are read from memory)

// Wavefronts a SIMD holds (workgroups a compute unit) and steps a wavefront keeps in flight. Measured on MI355X: three
// workgroups a unit (fewer registers each) and four steps in flight both stream less (the memory system is saturated by
// two and two; more concurrent streams cost DRAM locality).
constexpr int kMfmaWaves = 2;
constexpr int kMfmaTiles = 2;

// The launch: as many workgroups as the card holds at once, each working through units of the list (row, KV head
// group, query tile, partition) until it is exhausted. The hardware's own dispatcher binds a workgroup to an XCD by its
// id and starts workgroups strictly in order, so with units as uneven as ragged contexts make them it leaves slots
// idle behind a busy one; resident workgroups that pull the next unit themselves from the launch's counter (the
// caller's memory) keep every slot busy to the end. A workgroup knows its next unit while it works on the current one
// (its first two units are its index and that plus the grid; a ticket names the unit after the next): the next unit's
// page table entries are requested before the current unit's steps, its first keys, values and queries right after the
// current unit's last step, so the current unit's fold, its partials' stores and the draw of the following ticket
// happen while the next unit's rows are already on their way. A drawn unit without work (the list is a grid over rows
// of different lengths) is passed over by the drawing thread at once. The last workgroup to finish zeroes the counters
// for the next launch that uses them. Without counters the units are dealt in turn.
// MASKED: draft trees and sliding windows. DH: 128-wide halves of a head (1: heads of 128; 2: heads of 256, whose rows
// are 512 bytes of 16-bit pages by themselves, so a wavefront serves one KV head: HW 1): twice the key pieces, query
// pieces, score products and output tiles, the same layouts otherwise; twice the registers too, so one workgroup a
// compute unit, which keeps as many bytes in flight as two of the narrower ones (a step's rows are twice as long).
// QT: query tiles a wavefront holds (windows of several columns, wide GQA groups): a step's keys and values, once in
// the registers, are multiplied with each tile's queries and probabilities in turn, every tile with its own softmax
// state and accumulators, so a tile's bits are what they are alone and the rows are read once for QT tiles instead of
// once a tile. More than one tile takes the registers of a second workgroup on the compute unit (one stays). Built for
// four tiles (or a window's two) of 128-wide heads over 16-bit pages and two over 8-bit pages (pairs still fit two
// workgroups a compute unit), where it measured faster (64 rows ~U[1024, 8192] of 32 / 8 heads, 8 columns: 676 -> 480 us, FP8 376 -> 224);
// pairs of tiles of 256-wide heads keep one step in flight a wavefront instead of two (NT), or their registers spill;
// four tiles of 8-bit pages measured slower.
// NARROW: 64-wide heads, read as 128-wide ones. Two adjacent KV heads' rows of a position are 128 contiguous values,
// which is what a 128-wide head's row is: the launcher hands the kernel half the KV heads at twice the width and GQA
// groups twice as large (a group's first half the query heads of the even KV head, its second half the odd one's: the
// query heads' own order). A query row enters the first product with zeros in the other head's 64 dims (exact: the
// products with them are zeros), so its scores are its own head's; the second product gives it 128 output dims of
// which its own head's 64 are kept. Twice the matrix work a byte, on a pipe this kernel leaves nine tenths idle, for
// the 128-wide kernel's loads: 512 contiguous bytes a position and wavefront. What follows a KV head (row scales, an
// FP8 pool's multipliers) is looked up by the column's own head.
template <int KIND, bool F16, int HW, bool FUSED, bool MASKED, int DH = 1, int QT = 1, bool NARROW = false>
__global__ __launch_bounds__(256, (DH == 2 || QT > 2) ? 1 : kMfmaWaves) void attend_mfma_kernel(AttendArgs a) {
    static_assert(!NARROW || (DH == 1 && QT == 1), "64-wide heads: one 128-wide pair a tile row, one tile a workgroup");
    constexpr int NT = DH == 2 && QT == 2 ? 1 : kMfmaTiles;
    constexpr int D = 128 * DH;
    static_assert(DH == 1 || (DH == 2 && HW == 1), "heads of 128 or 256; one KV head a wavefront at 256");
    static_assert(QT == 1 || !FUSED, "several query tiles: the split launch");
    constexpr int EB = KIND == 0 ? 2 : 1;
    constexpr int CPH = kTileRows / HW;      // tile columns a KV head holds
    constexpr int SPW = kTileRows / HW;      // positions a wavefront's step covers (tile rows a KV head holds)
    constexpr int EPT = kTileRows * D / 256; // output elements a thread folds
    __shared__ __align__(16) float s_acc[4][kTileRows][D];
    __shared__ float s_m[4][kTileRows], s_l[4][kTileRows];
    __shared__ int s_rows[kLdsRows][5];      // count, first position, table row, first token, first partial row
    __shared__ int s_before[kLdsRows + 1];   // the dense list: partitions but the last of the rows before row r
    __shared__ int s_wave_sum[4];
    __shared__ int s_key[kLdsRows], s_order[kLdsRows];      // the dense list: the rows by the size of their last partition
    __shared__ unsigned s_unit;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c16 = lane & 15, u4 = lane >> 4;
    const unsigned grid = gridDim.x;
    const bool pulled = a.ticket != nullptr;
    const int hgroups = a.hkv / HW;
    // The list of units. Launches of up to kLdsRows rows take the dense list: every row's partitions but its last, row
    // by row (each for every head group and tile), then every row's last partition (usually a partial piece: the
    // smallest units go last) - no unit without work beyond tiles a short window row does not fill. Larger launches
    // take the grid units_x x units_y, whose units without work are passed over as they are drawn.
    const bool dense = a.n_rows <= kLdsRows;
    const unsigned per_row = (unsigned)(hgroups * a.tiles);
    const int slot_bytes = a.hkv * D * EB;
    const bool tree = MASKED && (a.parents != nullptr || a.parents64 != nullptr);
    const int win = MASKED ? a.sliding : 0;

    // -- every row's descriptors, once per workgroup
    auto row_from_memory = [&](int r, int (&d)[5]) __attribute__((always_inline)) {
        const int count = a.counts ? a.counts[r] : a.columns;
        const int64_t first64 = a.firsts[r];
        d[0] = min(count, a.columns);
        d[1] = (int)(first64 < 0 ? 0 : (first64 > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : first64));
        d[2] = a.rows[(int64_t)r * a.rows_step];
        d[3] = a.starts[r];
        d[4] = a.offsets ? a.offsets[r] - a.offsets[0] : r * a.columns;
    };
    for (int r = tid; r < min(a.n_rows, kLdsRows); r += 256) {
        int d[5];
        row_from_memory(r, d);
#pragma unroll
        for (int i = 0; i < 5; ++i) s_rows[r][i] = d[i];
    }
    lds_barrier();
    // Partitions that hold positions of row r (of its last column): what its units divide.
    auto row_partitions = [&](int r) __attribute__((always_inline)) -> int {
        const int count = s_rows[r][0];
        if (count <= 0) return 0;
        if constexpr (FUSED) return 1;
        const int n_keys = min(s_rows[r][1] + count, a.max_keys);
        return min((n_keys + a.piece - 1) / a.piece, a.parts);
    };
    if (dense) {      // s_before[r] = sum over r' < r of max(partitions(r') - 1, 0): thread i sums rows 2 i and 2 i + 1
        const int r0 = 2 * tid, r1 = 2 * tid + 1;
        const int c0 = r0 < a.n_rows ? max(row_partitions(r0) - 1, 0) : 0, c1 = r1 < a.n_rows ? max(row_partitions(r1) - 1, 0) : 0;
        const int run = (int)wave_inclusive_sum((unsigned)(c0 + c1));      // inclusive prefix over the threads
        if (lane == 63) s_wave_sum[wave] = run;
        lds_barrier();
        int base = 0;
        for (int w = 0; w < wave; ++w) base += s_wave_sum[w];
        const int upto = base + run - (c0 + c1);      // rows before 2 i
        if (r0 <= a.n_rows) s_before[r0] = upto;
        if (r1 <= a.n_rows) s_before[r1] = upto + c0;
        if (tid == 255 && kLdsRows <= a.n_rows) s_before[kLdsRows] = upto + c0 + c1;
        // The rows' last partitions are taken largest first (a launch's tail is as long as its last units): positions
        // the last partition holds (more than a piece where partitions hold several pieces), ties by row.
        for (int r = tid; r < a.n_rows; r += 256) {
            const int count = s_rows[r][0];
            int key = -1;
            if (count > 0) {
                const int n_keys = min(s_rows[r][1] + count, a.max_keys);
                const int n_pieces = (n_keys + a.piece - 1) / a.piece;
                key = FUSED ? n_keys : (n_pieces > a.parts ? a.piece + 1 : n_keys - (n_pieces - 1) * a.piece);
            }
            s_key[r] = key;
        }
        lds_barrier();
        for (int r = tid; r < a.n_rows; r += 256) {
            int rank = r;
            if (a.n_rows <= 256) {      // (larger launches keep the rows' order: ranking them costs more than it returns)
                const int key = s_key[r];
                rank = 0;
                for (int o = 0; o < a.n_rows; ++o) {
                    const int other = s_key[o];
                    rank += (other > key || (other == key && o < r)) ? 1 : 0;
                }
            }
            s_order[rank] = r;
        }
        lds_barrier();
    }
    const unsigned phase1 = dense ? (unsigned)__builtin_amdgcn_readfirstlane(s_before[a.n_rows]) * per_row : 0u;
    const unsigned total = dense ? phase1 + (unsigned)a.n_rows * per_row : (unsigned)a.units_x * (unsigned)a.units_y;

    // -- a unit of the list, decoded (everything uniform over the workgroup)
    struct Unit {
        bool valid;
        int kvh0, j0, b, count, first, n_keys, n_pieces, start, c_lo, prow;
        int64_t trow;
    };
    auto decode = [&](unsigned unit) __attribute__((always_inline)) -> Unit {
        Unit un;
        un.valid = false;
        if (unit >= total) return un;
        int bx, b, r;
        bool last = false;      // dense list: the row's last partition
        if (dense) {
            if (unit < phase1) {
                const int q = (int)(unit / per_row);      // the q-th of all rows' partitions but their last
                bx = (int)(unit % per_row);
                int lo = 0, hi = a.n_rows;                // the row: s_before[r] <= q < s_before[r + 1]
                while (hi - lo > 1) {
                    const int mid = (lo + hi) >> 1;
                    if (__builtin_amdgcn_readfirstlane(s_before[mid]) <= q) lo = mid;
                    else hi = mid;
                }
                r = lo, b = q - __builtin_amdgcn_readfirstlane(s_before[lo]);
            } else {
                const unsigned rest = unit - phase1;
                r = __builtin_amdgcn_readfirstlane(s_order[rest / per_row]), bx = (int)(rest % per_row), b = 0, last = true;
            }
        } else {
            bx = (int)(unit % (unsigned)a.units_x);
            b = (int)(unit / (unsigned)a.units_x);
            r = bx / (int)per_row;
            bx %= (int)per_row;
        }
        const int tile = bx % a.tiles;
        un.kvh0 = (bx / a.tiles) * HW;      // the first of the wavefronts' KV heads
        int d[5];
        if (r < kLdsRows) {
#pragma unroll
            for (int i = 0; i < 5; ++i) d[i] = s_rows[r][i];
        } else {
            row_from_memory(r, d);
        }
#pragma unroll
        for (int i = 0; i < 5; ++i) d[i] = __builtin_amdgcn_readfirstlane(d[i]);
        un.count = d[0], un.first = d[1], un.start = d[3], un.prow = d[4];
        un.trow = (int64_t)d[2] * a.tab_stride;
        un.j0 = tile * (QT * CPH);           // the first row of the unit's tiles in the flattened (column, group head) list
        if (un.j0 >= un.count * a.g) return un;
        un.c_lo = un.j0 / a.g;
        const int c_hi = min(un.count, (un.j0 + QT * CPH - 1) / a.g + 1);
        un.n_keys = min(un.first + c_hi, a.max_keys);
        un.n_pieces = (un.n_keys + a.piece - 1) / a.piece;
        if constexpr (!FUSED) {
            // Units are taken in list order, y slowest, and a launch's tail is as long as its last units: the row's
            // last partition (usually a partial piece, the smallest unit of work) is listed after every other
            // partition, in kTailClasses rows of y by its size (a whole piece or more first, the smallest last).
            const int np = min(un.n_pieces, a.parts);
            if (np <= 0) return un;
            if (dense) {
                if (last) b = np - 1;
                else if (b >= np - 1) return un;      // (a tile of earlier columns that holds fewer pieces than the row's last)
            } else {
                int cls = 0;
                if (np == un.n_pieces) cls = min(kTailClasses - 1, (np * a.piece - un.n_keys) * kTailClasses / a.piece);
                if (b >= a.units_y - kTailClasses) {
                    if (b - (a.units_y - kTailClasses) != cls) return un;
                    b = np - 1;
                } else if (b >= np - 1) {
                    return un;
                }
            }
        } else if (dense && !last) {
            return un;
        }
        un.b = b;
        un.valid = true;
        return un;
    };

    // -- what a lane holds for the whole launch
    // Tile rows: row i is position i % SPW of the step, of head i / SPW. This lane's places in the three layouts:
    //   keys    its row c16;  values and scores  rows 4 u4 .. 4 u4 + 3.
    const int hsel = c16 / CPH;                                     // the head (of the wavefront's HW) of this lane's tile column
    const int k_head = c16 / SPW, k_pos = c16 % SPW;
    const int r_head = (4 * u4) / SPW, r_pos = (4 * u4) % SPW;      // (SPW is 8 or 16: a lane's four rows lie in one head)
    const bool mine = hsel == r_head;                               // this lane's scores are of its own column's head
    // Byte offsets of what this lane reads in a step, from the step's first slot and the unit's first head.
    const uint32_t kvo = (uint32_t)(k_pos * slot_bytes + k_head * D * EB + u4 * 16);
    uint32_t vvo[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) vvo[p] = (uint32_t)((r_pos + p) * slot_bytes + r_head * D * EB + c16 * 8 * EB);
    const uint32_t svo = (uint32_t)(r_pos * a.hkv + r_head);      // row-scaled kinds: the lane's first score row's scale

    // -- a wavefront's walk over a partition's steps: steps wave, wave + 4, ... of pieces part, part + parts, ...
    // (positions stay below 2^31: the launcher bounds partitions x piece)
    struct Walk {
        int pi, st;
    };
    auto walk_base = [&](const Unit& un, const Walk& w) __attribute__((always_inline)) -> int {
        if (w.st * SPW >= a.piece) return -1;
        const int base = w.pi * a.piece + w.st * SPW;
        return base < un.n_keys ? base : -1;
    };
    auto walk_advance = [&](const Unit& un, Walk& w) __attribute__((always_inline)) -> int {
        w.st += 4;
        if (w.st * SPW >= a.piece) w.pi += a.parts, w.st = wave;
        return walk_base(un, w);
    };
    auto entry = [&](const Unit& un, int base) __attribute__((always_inline)) -> int {     // the page table entry of a step (uniform over the wavefront)
        int pidx = base >> a.page_shift;
        pidx = pidx < a.tab_width ? pidx : a.tab_width - 1;
        return a.tables[un.trow + pidx];
    };
    // The first steps of a partition with their page table entries: NT steps to fill the buffers and the NT after them.
    struct Lead {
        int base[2 * NT], e[2 * NT];
        Walk w;
    };
    auto lead_of = [&](const Unit& un, int part) __attribute__((always_inline)) -> Lead {
        Lead f;
        f.w.pi = part, f.w.st = wave;
        if (win > 0) {      // pieces wholly below the tile's window are skipped (no row sees them)
            const int wlo = un.first + un.c_lo - win + 1;
            const int below = (wlo > 0 ? wlo : 0) / a.piece - part;
            if (below > 0) f.w.pi = part + (below + a.parts - 1) / a.parts * a.parts;
        }
        f.base[0] = walk_base(un, f.w);
        const int again = f.base[0] >= 0 ? f.base[0] : 0;      // (a wavefront without a step reads position 0's entry)
        f.e[0] = entry(un, again);
#pragma unroll
        for (int i = 1; i < 2 * NT; ++i) {
            f.base[i] = f.base[i - 1] >= 0 ? walk_advance(un, f.w) : -1;
            f.e[i] = entry(un, f.base[i] >= 0 ? f.base[i] : again);
        }
        return f;
    };
    // A step's positions lie in one page (pages are powers of two from 16 up): its first slot, uniform.
    auto first_slot = [&](int base, int e) __attribute__((always_inline)) -> int64_t {
        return (int64_t)__builtin_amdgcn_readfirstlane(e) * a.page + (base & (a.page - 1));
    };
    // Loads of one step from its first slot. Every lane loads its place of the step whether the row holds that
    // position or not (the page does; a step past the row's keys is never listed): what such a place holds is dropped
    // where it is used (keys: the score is masked; values and scales: zeroed, see sanitize()).
    // (NARROW: `odd`, whether this lane's column is a query row of the pair's odd KV head; the scales are per KV head)
    auto fetch_k = [&](const Unit& un, int64_t slot0, Tile<KIND, DH>& t, int odd) __attribute__((always_inline)) {
        const uint8_t* sbase = a.kp + slot0 * slot_bytes + un.kvh0 * D * EB;
#pragma unroll
        for (int c = 0; c < (KIND == 0 ? 4 : 2) * DH; ++c) t.k[c] = *reinterpret_cast<const u32x4*>(sbase + kvo + 64 * c);
        if constexpr (KIND >= 2) {
            const int heads = NARROW ? 2 * a.hkv : a.hkv;      // scales a slot
            const int first = NARROW ? (int)svo * 2 + odd : (int)svo;      // (svo = r_pos * hkv + r_head)
            const float* ks = a.ks + slot0 * heads + (NARROW ? 2 * un.kvh0 : un.kvh0);
            const float* vs = a.vs + slot0 * heads + (NARROW ? 2 * un.kvh0 : un.kvh0);
#pragma unroll
            for (int i = 0; i < 4; ++i) t.ks[i] = ks[first + i * heads], t.vs[i] = vs[first + i * heads];
        }
    };
    // NARROW: whether this lane's tile column (a query row of the flattened list) belongs to the pair's odd KV head.
    auto odd_of = [&](const Unit& un) __attribute__((always_inline)) -> int {
        if constexpr (!NARROW) return 0;
        return ((un.j0 + c16 % CPH) % a.g) >= (a.g >> 1) ? 1 : 0;
    };
    auto fetch_v = [&](const Unit& un, int64_t slot0, Tile<KIND, DH>& t) __attribute__((always_inline)) {
        const uint8_t* sbase = a.vp + slot0 * slot_bytes + un.kvh0 * D * EB;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
#pragma unroll
            for (int h = 0; h < DH; ++h)
                t.v[p][h] = __builtin_nontemporal_load(reinterpret_cast<const typename Tile<KIND, DH>::VVec*>(sbase + vvo[p] + h * 128 * EB));
        }
    };

    // -- what a lane holds for one unit: its tile column's token, query head, last visible position, ancestors, scale,
    // and the query operand (its column's row, piece c = the dims the keys' piece c holds; zeros in a dead column)
    int col[QT], lim[QT];
    unsigned long long anc[QT];
#pragma unroll
    for (int q = 0; q < QT; ++q) col[q] = 0, lim[q] = -1, anc[q] = 0ull;
    float sscale = a.sscale;
    float vm_cur[HW], vm_nxt[HW];      // FP8 pages: the value multipliers of the unit's heads (requested with its queries, not in its fold)
#pragma unroll
    for (int h = 0; h < HW; ++h) vm_cur[h] = vm_nxt[h] = 1.0f;
    u32x4 qb[QT][4 * DH];
    auto value_multipliers = [&](const Unit& un) __attribute__((always_inline)) {      // (requested with the unit's page table entries)
        if constexpr (KIND == 1) {
#pragma unroll
            for (int h = 0; h < HW; ++h) vm_nxt[h] = a.hm ? a.hm[a.hkv + un.kvh0 + h] : a.v_mult;
        }
    };
    auto lane_values = [&](const Unit& un) __attribute__((always_inline)) {
        const int odd = odd_of(un);
        if constexpr (KIND == 1) sscale = a.sscale * (a.hm ? a.hm[NARROW ? 2 * (un.kvh0 + hsel) + odd : un.kvh0 + hsel] : a.k_mult);
#pragma unroll
        for (int q = 0; q < QT; ++q) {
            const int jr = un.j0 + q * CPH + c16 % CPH;
            col[q] = jr / a.g;
            const bool live = col[q] < un.count;
            const int qhead = (un.kvh0 + hsel) * a.g + jr % a.g;
            lim[q] = live ? min(un.first + col[q], un.n_keys - 1) : -1;
            anc[q] = (tree && live) ? ancestors(a, un.start, col[q]) : 0ull;
            const uint8_t* row = a.q + ((int64_t)(un.start + col[q]) * a.q_st + (int64_t)qhead * a.q_sh) * 2;
#pragma unroll
            for (int c = 0; c < 4 * DH; ++c) {
                // 16-bit pages: dims 32 c + 8 u4 ..; 8-bit pages: dims 64 (c / 2) + 16 u4 + 8 (c % 2) .. (the codes a lane's two loads hold)
                const int dim = KIND == 0 ? 32 * c + 8 * u4 : 64 * (c / 2) + 16 * u4 + 8 * (c % 2);
                qb[q][c] = u32x4{0, 0, 0, 0};
                if constexpr (NARROW) {      // the column's own head's 64 dims, zeros in the other head's
                    if (live && (dim >> 6) == odd) qb[q][c] = *reinterpret_cast<const u32x4*>(row + (dim & 63) * 2);
                } else {
                    if (live) qb[q][c] = *reinterpret_cast<const u32x4*>(row + dim * 2);
                }
            }
        }
    };

    Tile<KIND, DH> t[NT];
    auto fill = [&](const Unit& un, const Lead& f) __attribute__((always_inline)) {      // a partition's first NT steps
        const int again = f.base[0] >= 0 ? f.base[0] : 0;
        const int odd = odd_of(un);
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            const int64_t slot = first_slot(f.base[i] >= 0 ? f.base[i] : again, f.e[i]);
            fetch_k(un, slot, t[i], odd), fetch_v(un, slot, t[i]);
        }
    };

    unsigned u_next = blockIdx.x + grid;
    Unit cur = decode(blockIdx.x);
    Lead lead_cur;
    if (cur.valid) {
        lead_cur = lead_of(cur, FUSED ? 0 : cur.b);
        value_multipliers(cur);
        fill(cur, lead_cur);
        lane_values(cur);
#pragma unroll
        for (int h = 0; h < HW; ++h) vm_cur[h] = vm_nxt[h];
    }
    for (;;) {
        // The next unit: its first steps' page table entries are requested now and wait in registers.
        const Unit nxt = decode(u_next);
        Lead lead_nxt = {};
        if (nxt.valid) {
            lead_nxt = lead_of(nxt, FUSED ? 0 : nxt.b);
            value_multipliers(nxt);
        }
        // The ticket of the unit after the next is drawn when the current unit's steps are done (a returning atomic
        // in flight beside a unit's loads makes the waits on them coarser) and looked at after its fold.
        unsigned drawn = 0;
        bool sent = false;      // the next unit's first loads are out, the ticket is drawn
        auto hand_over = [&]() __attribute__((always_inline)) {
            if (pulled && tid == 0) drawn = atomicAdd(a.ticket, 1u);
            if (nxt.valid) {
                fill(nxt, lead_nxt);
                lane_values(nxt);
            }
            sent = true;
        };

        if (cur.valid) {
            const int part_lo = FUSED ? 0 : cur.b;
            const int part_hi = FUSED ? min(a.parts, cur.n_pieces) : cur.b + 1;
            float run_m[FUSED ? EPT : 1], run_l[FUSED ? EPT : 1], run_a[FUSED ? EPT : 1];
#pragma unroll
            for (int e = 0; e < (FUSED ? EPT : 1); ++e) run_m[e] = -INFINITY, run_l[e] = 0.0f, run_a[e] = 0.0f;
            for (int part = part_lo; part < part_hi; ++part) {
                float m[QT], l[QT];                  // the lane's column of each tile: running maximum (the same in its four lanes), the lane's share of the sum
                f32x4 acc[QT][8 * DH];               // O^T: acc[q][8 h + j][i] = dim 128 h + 32 u4 + 8 i + j of the lane's column of tile q
#pragma unroll
                for (int q = 0; q < QT; ++q) {
                    m[q] = -INFINITY, l[q] = 0.0f;
#pragma unroll
                    for (int j = 0; j < 8 * DH; ++j) acc[q][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                }

                auto step = [&](int base, Tile<KIND, DH>& tl, auto&& refill_k, auto&& refill_v) __attribute__((always_inline)) {
                    if (base + SPW > cur.n_keys) {
                        // The row's last step: what lies past its keys may be anything, and a probability of zero
                        // times a NaN is a NaN.
#pragma unroll
                        for (int p = 0; p < 4; ++p) {
                            if (base + r_pos + p >= cur.n_keys) {
#pragma unroll
                                for (int h = 0; h < DH; ++h) {
                                    if constexpr (KIND == 0) tl.v[p][h] = u32x4{0, 0, 0, 0};
                                    else tl.v[p][h] = u32x2{0, 0};
                                }
                                if constexpr (KIND >= 2) tl.vs[p] = 0.0f;
                            }
                        }
                    }
                    // -- scores
                    u32x4 ka[4 * DH];
                    if constexpr (KIND == 0) {
#pragma unroll
                        for (int c = 0; c < 4 * DH; ++c) ka[c] = tl.k[c];
                    } else {
#pragma unroll
                        for (int c = 0; c < 4 * DH; ++c) {
                            const uint32_t w0 = c % 2 ? tl.k[c / 2].z : tl.k[c / 2].x, w1 = c % 2 ? tl.k[c / 2].w : tl.k[c / 2].y;
                            const u32x2 lo = codes4_to_pairs<KIND>(w0), hi = codes4_to_pairs<KIND>(w1);
                            ka[c] = u32x4{lo.x, lo.y, hi.x, hi.y};
                        }
                    }
                    f32x4 s0[QT], s1[QT];
#pragma unroll
                    for (int q = 0; q < QT; ++q) {
                        s0[q] = mfma_k32<F16>(ka[0], qb[q][0], f32x4{0.0f, 0.0f, 0.0f, 0.0f});
                        s1[q] = mfma_k32<F16>(ka[1], qb[q][1], f32x4{0.0f, 0.0f, 0.0f, 0.0f});
                    }
#pragma unroll
                    for (int c = 2; c < 4 * DH; c += 2) {      // (two chains, the even pieces and the odd ones)
#pragma unroll
                        for (int q = 0; q < QT; ++q) {
                            s0[q] = mfma_k32<F16>(ka[c], qb[q][c], s0[q]);
                            s1[q] = mfma_k32<F16>(ka[c + 1], qb[q][c + 1], s1[q]);
                        }
                    }
                    float ks4[4], vs4[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) ks4[i] = KIND >= 2 ? tl.ks[i] : 1.0f, vs4[i] = KIND >= 2 ? tl.vs[i] : 1.0f;
                    refill_k();      // (the keys' registers are free: the loads of NT steps ahead go out)
                    u32x2 pb[QT];
#pragma unroll
                    for (int q = 0; q < QT; ++q) {
                        // the lane's scores: its column at positions base + r_pos + i of head r_head; another head's column sees nothing
                        const int room = lim[q] - (base + r_pos);      // visible while i <= room
                        float x[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            x[i] = (s0[q][i] + s1[q][i]) * (KIND >= 2 ? sscale * ks4[i] : sscale);
                            bool vis = mine && i <= room;
                            if constexpr (MASKED) {
                                const int n = base + r_pos + i;
                                if (tree) vis = vis && (n < cur.first || ((anc[q] >> ((n - cur.first) & 63)) & 1ull) != 0);
                                if (win > 0) vis = vis && n > cur.first + col[q] - win;
                            }
                            x[i] = vis ? x[i] : -INFINITY;
                        }
                        const float top = max_across_quarters(__builtin_fmaxf(__builtin_fmaxf(x[0], x[1]), __builtin_fmaxf(x[2], x[3])));
                        const float m_new = __builtin_fmaxf(m[q], top);
                        const float sub = m_new == -INFINITY ? 0.0f : m_new;
                        const float alpha = m[q] == -INFINITY ? 1.0f : exp2_fast(m[q] - sub);      // (nothing summed yet: nothing to rescale)
                        float p[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) p[i] = exp2_fast(x[i] - sub);
                        l[q] = __builtin_fmaf(l[q], alpha, (p[0] + p[1]) + (p[2] + p[3]));
                        m[q] = m_new;
                        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {     // some row's maximum moved: rescale
#pragma unroll
                            for (int j = 0; j < 8 * DH; ++j) acc[q][j] *= alpha;
                        }
                        pb[q] = u32x2{pair16<F16>(p[0] * vs4[0], p[1] * vs4[1]), pair16<F16>(p[2] * vs4[2], p[3] * vs4[3])};
                    }
                    // -- values: dims {8 i + j} of the lane's four rows as two 16-bit pairs (one v_perm each), then O^T += V^T P^T
#pragma unroll
                    for (int h = 0; h < DH; ++h) {
                    if constexpr (KIND == 0) {
#pragma unroll
                        for (int w = 0; w < 4; ++w) {
                            const u32x2 lo = {__builtin_amdgcn_perm(tl.v[1][h][w], tl.v[0][h][w], 0x05040100), __builtin_amdgcn_perm(tl.v[3][h][w], tl.v[2][h][w], 0x05040100)};
                            const u32x2 hi = {__builtin_amdgcn_perm(tl.v[1][h][w], tl.v[0][h][w], 0x07060302), __builtin_amdgcn_perm(tl.v[3][h][w], tl.v[2][h][w], 0x07060302)};
#pragma unroll
                            for (int q = 0; q < QT; ++q) {
                                acc[q][8 * h + 2 * w] = mfma_k16<F16>(lo, pb[q], acc[q][8 * h + 2 * w]);
                                acc[q][8 * h + 2 * w + 1] = mfma_k16<F16>(hi, pb[q], acc[q][8 * h + 2 * w + 1]);
                            }
                        }
                    } else {
#pragma unroll
                        for (int w = 0; w < 2; ++w) {
                            // bytes (a0 b0 a1 b1) and (a2 b2 a3 b3): two rows' codes of one dim side by side
                            const uint32_t lo01 = __builtin_amdgcn_perm(tl.v[1][h][w], tl.v[0][h][w], 0x05010400), hi01 = __builtin_amdgcn_perm(tl.v[1][h][w], tl.v[0][h][w], 0x07030602);
                            const uint32_t lo23 = __builtin_amdgcn_perm(tl.v[3][h][w], tl.v[2][h][w], 0x05010400), hi23 = __builtin_amdgcn_perm(tl.v[3][h][w], tl.v[2][h][w], 0x07030602);
                            // (dims 4 w + 0, 1 from the low halves, 2, 3 from the high ones; .x: rows 0, 1; .y: rows 2, 3)
                            const u32x2 a01 = codes4_to_pairs<KIND>(lo01), a23 = codes4_to_pairs<KIND>(lo23);
                            const u32x2 b01 = codes4_to_pairs<KIND>(hi01), b23 = codes4_to_pairs<KIND>(hi23);
                            const u32x2 va[4] = {u32x2{a01.x, a23.x}, u32x2{a01.y, a23.y}, u32x2{b01.x, b23.x}, u32x2{b01.y, b23.y}};
#pragma unroll
                            for (int q = 0; q < QT; ++q) {
#pragma unroll
                                for (int j = 0; j < 4; ++j) acc[q][8 * h + 4 * w + j] = mfma_k16<F16>(va[j], pb[q], acc[q][8 * h + 4 * w + j]);
                            }
                        }
                    }
                    }
                    refill_v();
                };

                // Software pipeline over NT steps: a step's keys are reloaded (for NT steps ahead) as soon as its
                // scores are issued, its values as soon as its second product is; the page table entries run NT steps
                // further ahead. While the NT steps ahead all exist the loop's loads are unconditional (exact waits);
                // the wavefront's last steps are peeled: no step is loaded that is not used (a re-read of an earlier
                // step would come from HBM again: the caches have long turned over).
                Lead f = lead_cur;
                const int odd_cur = odd_of(cur);
                if (part != part_lo) {
                    f = lead_of(cur, part);
                    fill(cur, f);
                }
                if (f.base[0] >= 0) {
                    const int again = f.base[0];
                    int at[NT], ahead[NT], e_ahead[NT];
#pragma unroll
                    for (int i = 0; i < NT; ++i) at[i] = f.base[i], ahead[i] = f.base[NT + i], e_ahead[i] = f.e[NT + i];
                    while (ahead[NT - 1] >= 0) {
#pragma unroll
                        for (int i = 0; i < NT; ++i) {
                            const int after = walk_advance(cur, f.w);      // NT steps past the one this buffer is refilled with
                            const int e_after = entry(cur, after >= 0 ? after : again);
                            const int64_t slot = first_slot(ahead[i], e_ahead[i]);
                            step(at[i], t[i], [&]() __attribute__((always_inline)) { fetch_k(cur, slot, t[i], odd_cur); },
                                 [&]() __attribute__((always_inline)) { fetch_v(cur, slot, t[i]); });
                            at[i] = ahead[i], ahead[i] = after, e_ahead[i] = e_after;
                        }
                    }
#pragma unroll
                    for (int i = 0; i < NT; ++i) {
                        if (at[i] >= 0) {
                            const bool again_i = ahead[i] >= 0;
                            const int64_t slot = first_slot(again_i ? ahead[i] : again, e_ahead[i]);
                            step(at[i], t[i], [&]() __attribute__((always_inline)) { if (again_i) fetch_k(cur, slot, t[i], odd_cur); },
                                 [&]() __attribute__((always_inline)) { if (again_i) fetch_v(cur, slot, t[i]); });
                        }
                    }
#pragma unroll
                    for (int i = 0; i < NT; ++i) {
                        if (ahead[i] >= 0) step(ahead[i], t[i], []() {}, []() {});
                    }
                }
                // The unit's steps are done: the next unit's first keys, values and queries go out before the fold.
                const int fold_col_j0 = cur.j0, fold_kvh0 = cur.kvh0;
                if (part == part_hi - 1) hand_over();

                // A tile's column sums over its four lanes, then the four wavefronts through LDS, in wavefront order; tile
                // after tile through the same arrays.
#pragma unroll
                for (int q = 0; q < QT; ++q) {
                const float l_col = sum_across_quarters(l[q]);
                if (part != part_lo || q > 0) lds_barrier();      // the fold before has read the LDS
#pragma unroll
                for (int h = 0; h < DH; ++h) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        *reinterpret_cast<f32x4*>(&s_acc[wave][c16][128 * h + 32 * u4 + 8 * i]) = f32x4{acc[q][8 * h][i], acc[q][8 * h + 1][i], acc[q][8 * h + 2][i], acc[q][8 * h + 3][i]};
                        *reinterpret_cast<f32x4*>(&s_acc[wave][c16][128 * h + 32 * u4 + 8 * i + 4]) = f32x4{acc[q][8 * h + 4][i], acc[q][8 * h + 5][i], acc[q][8 * h + 6][i], acc[q][8 * h + 7][i]};
                    }
                }
                if (u4 == 0) s_m[wave][c16] = m[q], s_l[wave][c16] = l_col;
                lds_barrier();
#pragma unroll
                for (int e = 0; e < EPT; ++e) {
                    const int idx = tid + e * 256;
                    const int cc = idx / D, d = idx % D;
                    const int head_i = cc / CPH;
                    const int j = fold_col_j0 + q * CPH + cc % CPH;
                    const int c = j / a.g;
                    float M = s_m[0][cc];
#pragma unroll
                    for (int w = 1; w < 4; ++w) M = __builtin_fmaxf(M, s_m[w][cc]);
                    const float sub = M == -INFINITY ? 0.0f : M;
                    float L = 0.0f, A = 0.0f;
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const float fw = exp2_fast(s_m[w][cc] - sub);
                        L = __builtin_fmaf(s_l[w][cc], fw, L);
                        A = __builtin_fmaf(s_acc[w][cc][d], fw, A);
                    }
                    // NARROW: the element is kept where its dim lies in the 64 of its column's own KV head
                    const int odd = NARROW ? ((j % a.g) >= (a.g >> 1) ? 1 : 0) : 0;
                    const bool kept = !NARROW || (d >> 6) == odd;
                    if constexpr (KIND == 1) {
                        if constexpr (NARROW) A *= a.hm ? a.hm[2 * a.hkv + 2 * (fold_kvh0 + head_i) + odd] : a.v_mult;
                        else A *= HW == 1 ? vm_cur[0] : (head_i == 0 ? vm_cur[0] : vm_cur[HW - 1]);
                    }
                    if (c < cur.count && kept) {
                        if constexpr (FUSED) {
                            // A column folds the partitions that hold its positions, as the merge does.
                            const int held = min(a.parts, (min(cur.first + c + 1, a.max_keys) + a.piece - 1) / a.piece);
                            if (part < held) {
                                const Fold fo = fold(run_m[e], run_l[e], M, L);
                                run_a[e] = __builtin_fmaf(run_a[e], fo.keep, A * fo.take);
                                run_m[e] = fo.m, run_l[e] = fo.l;
                            }
                        } else {
                            const int64_t at = ((int64_t)(cur.prow + c) * a.hq + (fold_kvh0 + head_i) * a.g + j % a.g) * a.parts + cur.b;
                            if constexpr (NARROW) a.po[at * 64 + (d & 63)] = A;
                            else a.po[at * D + d] = A;
                            if ((d & (NARROW ? 63 : D - 1)) == 0) a.pm[at] = M, a.pl[at] = L;
                        }
                    }
                }
                }
            }
            if constexpr (FUSED) {
#pragma unroll
                for (int e = 0; e < EPT; ++e) {
                    const int idx = tid + e * 256;
                    const int cc = idx / D, d = idx % D;
                    const int j = cur.j0 + cc % CPH;
                    const int c = j / a.g;
                    const bool kept = !NARROW || (d >> 6) == ((j % a.g) >= (a.g >> 1) ? 1 : 0);
                    if (c < cur.count && kept) {
                        const int head = (cur.kvh0 + cc / CPH) * a.g + j % a.g;
                        float M = run_m[e], L = run_l[e], A = run_a[e];
                        if (a.sinks) {
                            const Fold fo = fold(M, L, a.sinks[head] * kLog2e, 1.0f);
                            A *= fo.keep, M = fo.m, L = fo.l;
                        }
                        const float o = L != 0.0f ? A / L : 0.0f;
                        store_out(a.out, a.out_dtype, (int64_t)(cur.start + c) * a.o_st + (int64_t)head * a.o_sh + (NARROW ? (d & 63) : d), o);
                        if (a.lse && (d & (NARROW ? 63 : D - 1)) == 0) a.lse[(int64_t)(cur.start + c) * a.hq + head] = L != 0.0f ? __builtin_fmaf(M, kLn2, __logf(L)) : -INFINITY;
                    }
                }
            }
        }
        if (!sent) hand_over();      // (nothing to do in this round: the next unit's first rows go out all the same)

        // The unit after the next: the ticket drawn above, or, while it names a unit without work, the ones after it.
        unsigned u_after = u_next + grid;
        if (pulled) {
            if (tid == 0) {
                unsigned found = 2 * grid + drawn;
                while (found < total && !decode(found).valid) found = 2 * grid + atomicAdd(a.ticket, 1u);
                s_unit = found;
            }
            lds_barrier();      // (and every thread is done with the fold's shared arrays)
            u_after = s_unit;
        } else {
            lds_barrier();
        }
        if (!nxt.valid && u_next >= total && u_after >= total) break;
        cur = nxt, lead_cur = lead_nxt;
#pragma unroll
        for (int h = 0; h < HW; ++h) vm_cur[h] = vm_nxt[h];
        u_next = u_after;
        lds_barrier();      // every thread has read s_unit before the next round's draw is published
    }
    if (!pulled) return;
    if (threadIdx.x == 0) {
        if (atomicAdd(a.ticket + 1, 1u) == grid - 1) {
            atomicExch(a.ticket, 0u);
            atomicExch(a.ticket + 1, 0u);
        }
    }
}

}   // namespace pkv
