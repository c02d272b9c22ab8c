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

template <int KIND>
struct Tile {
    using VVec = typename std::conditional<KIND == 0, u32x4, u32x2>::type;
    u32x4 k[KIND == 0 ? 4 : 2];      // the lane's pieces of its position's K row
    VVec v[4];                        // the lane's 8 dims of the V rows of its quarter's four positions
    float ks[KIND >= 2 ? 4 : 1], vs[KIND >= 2 ? 4 : 1];      // row-scaled kinds: the scales of positions 4 u .. 4 u + 3
};

constexpr int kTileRows = 16;      // query rows (columns of S^T) a tile holds

// One unit of work: (ux, uy) of a units_x x units_y list. MASKED: draft trees and sliding windows.
template <int KIND, bool F16, int HW, bool FUSED, bool MASKED, int NT>
PKV_DEV void attend_mfma_unit(const AttendArgs& a, const int ux, const int uy, float (&s_acc)[4][kTileRows][128],
                              float (&s_m)[4][kTileRows], float (&s_l)[4][kTileRows]) {
    constexpr int D = 128;
    constexpr int EB = KIND == 0 ? 2 : 1;
    constexpr int CPH = kTileRows / HW;      // tile columns a KV head holds
    constexpr int SPW = kTileRows / HW;      // positions a wavefront's step covers (tile rows a KV head holds)
    constexpr int EPT = kTileRows * D / 256; // output elements a thread folds
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c16 = lane & 15, u = lane >> 4;
    int bx = ux;
    const int tile = bx % a.tiles;
    bx /= a.tiles;
    const int hgroups = a.hkv / HW;
    const int kvh0 = (bx % hgroups) * HW;      // the first of the wavefront's KV heads
    const int r = bx / hgroups;
    int b = uy;
    // The row's descriptors are read together, ahead of every test that could end the unit: one memory round trip.
    int count_raw = *(a.counts ? a.counts + r : a.starts + r);      // (no load under a condition)
    int64_t first64 = a.firsts[r];
    int table_row = a.rows[(int64_t)r * a.rows_step];
    int start = a.starts[r];
    int off_r = *(a.offsets ? a.offsets + r : a.starts + r), off_0 = *(a.offsets ? a.offsets : a.starts);
    asm volatile("" : "+v"(count_raw), "+v"(first64), "+v"(table_row), "+v"(start), "+v"(off_r), "+v"(off_0));
    count_raw = __builtin_amdgcn_readfirstlane(count_raw), table_row = __builtin_amdgcn_readfirstlane(table_row);
    start = __builtin_amdgcn_readfirstlane(start), off_r = __builtin_amdgcn_readfirstlane(off_r), off_0 = __builtin_amdgcn_readfirstlane(off_0);
    first64 = (int64_t)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(first64 >> 32)) << 32) |
                        (uint32_t)__builtin_amdgcn_readfirstlane((int)first64));
    const int64_t prow = a.offsets ? (int64_t)(off_r - off_0) : (int64_t)r * a.columns;      // the row's first partial row
    const int count = min(a.counts ? count_raw : a.columns, a.columns);
    const int64_t trow = (int64_t)table_row * a.tab_stride;
    const int j0 = tile * CPH;                  // the tile's first row of the flattened (column, group head) list
    if (j0 >= count * a.g) return;
    const int c_lo = j0 / a.g;
    const int c_hi = min(count, (j0 + CPH - 1) / a.g + 1);
    int64_t nk64 = first64 + c_hi;
    nk64 = nk64 < 0 ? 0 : (nk64 > (int64_t)a.max_keys ? (int64_t)a.max_keys : nk64);
    const int n_keys = (int)nk64;
    const int first = (int)(first64 < 0 ? 0 : (first64 > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : first64));
    const int n_pieces = (n_keys + a.piece - 1) / a.piece;
    if constexpr (!FUSED) {
        // Units are taken in list order, y slowest, and a launch's tail is as long as its last units: the row's last
        // partition (usually a partial piece, the smallest unit of work) is listed after every other partition, in
        // kTailClasses rows of y by its size (a whole piece or more first, the smallest remainders last).
        const int np = min(n_pieces, a.parts);
        if (np <= 0) return;
        int cls = 0;
        if (np == n_pieces) cls = min(kTailClasses - 1, (np * a.piece - n_keys) * kTailClasses / a.piece);
        if (b >= a.units_y - kTailClasses) {
            if (b - (a.units_y - kTailClasses) != cls) return;
            b = np - 1;
        } else if (b >= np - 1) {
            return;
        }
    }

    // This lane's tile column: which of the wavefront's heads it belongs to, its row of the list, its token's column
    // and the last position that column sees.
    const int hsel = c16 / CPH;
    const int jr = j0 + c16 % CPH;
    const int col = jr / a.g;
    const bool live = col < count;
    const int qhead = (kvh0 + hsel) * a.g + jr % a.g;
    const int lim = live ? min(first + col, n_keys - 1) : -1;
    const bool tree = MASKED && (a.parents != nullptr || a.parents64 != nullptr);
    const unsigned long long anc = (tree && live) ? ancestors(a, start, col) : 0ull;
    const int win = MASKED ? a.sliding : 0;
    // Tile rows: row i is position i % SPW of the step, of head i / SPW. This lane's places in the three layouts:
    //   keys    its row c16;  values and scores  rows 4 u .. 4 u + 3.
    const int k_head = c16 / SPW, k_pos = c16 % SPW;
    const int r_head = (4 * u) / SPW, r_pos = (4 * u) % SPW;      // (SPW is 8 or 16: a lane's four rows lie in one head)
    const bool mine = hsel == r_head;                               // this lane's scores are of its own column's head
    float sscale = a.sscale;
    if constexpr (KIND == 1) sscale *= a.hm ? a.hm[kvh0 + hsel] : a.k_mult;

    // Byte offsets of what this lane reads in a step, from the step's first slot; the same in every step.
    const int slot_bytes = a.hkv * D * EB;
    const uint32_t kvo = (uint32_t)(k_pos * slot_bytes + (kvh0 + k_head) * D * EB + u * 16);
    uint32_t vvo[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) vvo[p] = (uint32_t)((r_pos + p) * slot_bytes + (kvh0 + r_head) * D * EB + c16 * 8 * EB);
    const uint32_t svo = (uint32_t)(r_pos * a.hkv + kvh0 + r_head);      // row-scaled kinds: the lane's first score row's scale

    auto entry = [&](int base) __attribute__((always_inline)) -> int {     // the page table entry of a step (uniform over the wavefront)
        int pidx = base >> a.page_shift;
        pidx = pidx < a.tab_width ? pidx : a.tab_width - 1;
        return a.tables[trow + pidx];
    };
    // A step's positions lie in one page (pages are powers of two from 16 up): its first slot, uniform.
    auto first_slot = [&](int base, int e) __attribute__((always_inline)) -> int64_t {
        return (int64_t)__builtin_amdgcn_readfirstlane(e) * a.page + (base & (a.page - 1));
    };
    // Loads of one step from its first slot. Every lane loads its place of the step whether the row holds that
    // position or not (the page does; a step past the row's keys is never listed): what such a place holds is dropped
    // where it is used (keys: the score is masked; values and scales: zeroed, see sanitize()).
    auto fetch_k = [&](int64_t slot0, Tile<KIND>& t) __attribute__((always_inline)) {
        const uint8_t* sbase = a.kp + slot0 * slot_bytes;
        if constexpr (KIND == 0) {
#pragma unroll
            for (int c = 0; c < 4; ++c) t.k[c] = *reinterpret_cast<const u32x4*>(sbase + kvo + 64 * c);
        } else {
            t.k[0] = *reinterpret_cast<const u32x4*>(sbase + kvo);
            t.k[1] = *reinterpret_cast<const u32x4*>(sbase + kvo + 64);
        }
        if constexpr (KIND >= 2) {
            const float* ks = a.ks + slot0 * a.hkv;
            const float* vs = a.vs + slot0 * a.hkv;
#pragma unroll
            for (int i = 0; i < 4; ++i) t.ks[i] = ks[svo + i * a.hkv], t.vs[i] = vs[svo + i * a.hkv];
        }
    };
    auto fetch_v = [&](int64_t slot0, Tile<KIND>& t) __attribute__((always_inline)) {
        const uint8_t* sbase = a.vp + slot0 * slot_bytes;
#pragma unroll
        for (int p = 0; p < 4; ++p)
            t.v[p] = __builtin_nontemporal_load(reinterpret_cast<const typename Tile<KIND>::VVec*>(sbase + vvo[p]));
    };
    // The row's last step: what lies past its keys may be anything, and a probability of zero times a NaN is a NaN.
    auto sanitize = [&](int base, Tile<KIND>& t) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            if (base + r_pos + p >= n_keys) {
                if constexpr (KIND == 0) t.v[p] = u32x4{0, 0, 0, 0};
                else t.v[p] = u32x2{0, 0};
                if constexpr (KIND >= 2) t.vs[p] = 0.0f;
            }
        }
    };

    // A wavefront's walk over a partition's steps: steps wave, wave + 4, ... of pieces part, part + parts, ...
    // (positions stay below 2^31: the launcher bounds partitions x piece)
    int pi, st;
    auto start_part = [&](int part) __attribute__((always_inline)) {
        pi = part, st = wave;
        if (win > 0) {      // pieces wholly below the tile's window are skipped (no row sees them)
            const int wlo = first + c_lo - win + 1;
            const int below = (wlo > 0 ? wlo : 0) / a.piece - part;
            if (below > 0) pi = part + (below + a.parts - 1) / a.parts * a.parts;
        }
    };
    auto base_of = [&]() __attribute__((always_inline)) -> int {
        if (st * SPW >= a.piece) return -1;
        const int base = pi * a.piece + st * SPW;
        return base < n_keys ? base : -1;
    };
    auto advance = [&]() __attribute__((always_inline)) -> int {
        st += 4;
        if (st * SPW >= a.piece) pi += a.parts, st = wave;
        return base_of();
    };
    // The first steps of a partition with their page table entries: NT steps to fill the buffers and one ahead.
    struct Lead {
        int base[NT + 1], e[NT + 1];
    };
    auto lead_of = [&](int part) __attribute__((always_inline)) -> Lead {
        Lead f;
        start_part(part);
        f.base[0] = base_of();
        const int again = f.base[0] >= 0 ? f.base[0] : 0;      // (a wavefront without a step reads position 0's entry)
        f.e[0] = entry(again);
#pragma unroll
        for (int i = 1; i <= NT; ++i) {
            f.base[i] = f.base[i - 1] >= 0 ? advance() : -1;
            f.e[i] = entry(f.base[i] >= 0 ? f.base[i] : again);
        }
        return f;
    };
    const int part_lo = FUSED ? 0 : b;
    const int part_hi = FUSED ? min(a.parts, n_pieces) : b + 1;
    const Lead lead_first = lead_of(part_lo);

    // The query operand: this lane's column's row, piece c = the dims the keys' piece c holds (zeros in a dead column).
    u32x4 qb[4];
    {
        const uint8_t* row = a.q + ((int64_t)(start + col) * a.q_st + (int64_t)qhead * a.q_sh) * 2;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            // 16-bit pages: dims 32 c + 8 u ..; 8-bit pages: dims 64 (c / 2) + 16 u + 8 (c % 2) .. (the codes a lane's two loads hold)
            const int dim = KIND == 0 ? 32 * c + 8 * u : 64 * (c / 2) + 16 * u + 8 * (c % 2);
            qb[c] = u32x4{0, 0, 0, 0};
            if (live) qb[c] = *reinterpret_cast<const u32x4*>(row + dim * 2);
        }
    }
    float run_m[FUSED ? EPT : 1], run_l[FUSED ? EPT : 1], run_a[FUSED ? EPT : 1];
#pragma unroll
    for (int e = 0; e < (FUSED ? EPT : 1); ++e) run_m[e] = -INFINITY, run_l[e] = 0.0f, run_a[e] = 0.0f;

    for (int part = part_lo; part < part_hi; ++part) {
        float m = -INFINITY, l = 0.0f;      // the lane's column: running maximum (the same in its four lanes), the lane's share of the sum
        f32x4 acc[8];                        // O^T: acc[j][i] = dim 32 u + 8 i + j of the lane's column
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

        auto step = [&](int base, Tile<KIND>& t, auto&& refill_k, auto&& refill_v) __attribute__((always_inline)) {
            if (base + SPW > n_keys) sanitize(base, t);
            // -- scores
            u32x4 ka[4];
            if constexpr (KIND == 0) {
#pragma unroll
                for (int c = 0; c < 4; ++c) ka[c] = t.k[c];
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const uint32_t w0 = c % 2 ? t.k[c / 2].z : t.k[c / 2].x, w1 = c % 2 ? t.k[c / 2].w : t.k[c / 2].y;
                    const u32x2 lo = codes4_to_pairs<KIND>(w0), hi = codes4_to_pairs<KIND>(w1);
                    ka[c] = u32x4{lo.x, lo.y, hi.x, hi.y};
                }
            }
            f32x4 s0 = mfma_k32<F16>(ka[0], qb[0], f32x4{0.0f, 0.0f, 0.0f, 0.0f});
            f32x4 s1 = mfma_k32<F16>(ka[1], qb[1], f32x4{0.0f, 0.0f, 0.0f, 0.0f});
            s0 = mfma_k32<F16>(ka[2], qb[2], s0);
            s1 = mfma_k32<F16>(ka[3], qb[3], s1);
            float ks4[4], vs4[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) ks4[i] = KIND >= 2 ? t.ks[i] : 1.0f, vs4[i] = KIND >= 2 ? t.vs[i] : 1.0f;
            refill_k();      // (the keys' registers are free: the loads of NT steps ahead go out)
            // the lane's scores: its column at positions base + r_pos + i of head r_head; another head's column sees nothing
            const int room = lim - (base + r_pos);      // visible while i <= room
            float x[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                x[i] = (s0[i] + s1[i]) * (KIND >= 2 ? sscale * ks4[i] : sscale);
                bool vis = mine && i <= room;
                if constexpr (MASKED) {
                    const int n = base + r_pos + i;
                    if (tree) vis = vis && (n < first || ((anc >> ((n - first) & 63)) & 1ull) != 0);
                    if (win > 0) vis = vis && n > first + col - win;
                }
                x[i] = vis ? x[i] : -INFINITY;
            }
            const float top = max_across_quarters(__builtin_fmaxf(__builtin_fmaxf(x[0], x[1]), __builtin_fmaxf(x[2], x[3])));
            const float m_new = __builtin_fmaxf(m, top);
            const float sub = m_new == -INFINITY ? 0.0f : m_new;
            const float alpha = m == -INFINITY ? 1.0f : exp2_fast(m - sub);      // (nothing summed yet: nothing to rescale)
            float p[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) p[i] = exp2_fast(x[i] - sub);
            l = __builtin_fmaf(l, alpha, (p[0] + p[1]) + (p[2] + p[3]));
            m = m_new;
            if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {     // some row's maximum moved: rescale
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[j] *= alpha;
            }
            const u32x2 pb = {pair16<F16>(p[0] * vs4[0], p[1] * vs4[1]), pair16<F16>(p[2] * vs4[2], p[3] * vs4[3])};
            // -- values: dims {8 i + j} of the lane's four rows as two 16-bit pairs (one v_perm each), then O^T += V^T P^T
            if constexpr (KIND == 0) {
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const u32x2 lo = {__builtin_amdgcn_perm(t.v[1][w], t.v[0][w], 0x05040100), __builtin_amdgcn_perm(t.v[3][w], t.v[2][w], 0x05040100)};
                    const u32x2 hi = {__builtin_amdgcn_perm(t.v[1][w], t.v[0][w], 0x07060302), __builtin_amdgcn_perm(t.v[3][w], t.v[2][w], 0x07060302)};
                    acc[2 * w] = mfma_k16<F16>(lo, pb, acc[2 * w]);
                    acc[2 * w + 1] = mfma_k16<F16>(hi, pb, acc[2 * w + 1]);
                }
            } else {
#pragma unroll
                for (int w = 0; w < 2; ++w) {
                    // bytes (a0 b0 a1 b1) and (a2 b2 a3 b3): two rows' codes of one dim side by side
                    const uint32_t lo01 = __builtin_amdgcn_perm(t.v[1][w], t.v[0][w], 0x05010400), hi01 = __builtin_amdgcn_perm(t.v[1][w], t.v[0][w], 0x07030602);
                    const uint32_t lo23 = __builtin_amdgcn_perm(t.v[3][w], t.v[2][w], 0x05010400), hi23 = __builtin_amdgcn_perm(t.v[3][w], t.v[2][w], 0x07030602);
                    // (dims 4 w + 0, 1 from the low halves, 2, 3 from the high ones; .x: rows 0, 1; .y: rows 2, 3)
                    const u32x2 a01 = codes4_to_pairs<KIND>(lo01), a23 = codes4_to_pairs<KIND>(lo23);
                    const u32x2 b01 = codes4_to_pairs<KIND>(hi01), b23 = codes4_to_pairs<KIND>(hi23);
                    const u32x2 va[4] = {u32x2{a01.x, a23.x}, u32x2{a01.y, a23.y}, u32x2{b01.x, b23.x}, u32x2{b01.y, b23.y}};
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[4 * w + j] = mfma_k16<F16>(va[j], pb, acc[4 * w + j]);
                }
            }
            refill_v();
        };

        // Software pipeline over NT steps: a step's keys are reloaded (for NT steps ahead) as soon as its scores are
        // issued, its values as soon as its second product is; the page table entries run one step further ahead.
        // Past the wavefront's last step the loads re-read its first step (the caches hold it).
        Tile<KIND> t[NT];
        const Lead f = part == part_lo ? lead_first : lead_of(part);
        if (f.base[0] >= 0) {
            const int again = f.base[0];
            auto safe = [&](int base) __attribute__((always_inline)) { return base >= 0 ? base : again; };
            int cur[NT], next = f.base[NT], e_next = f.e[NT];
#pragma unroll
            for (int i = 0; i < NT; ++i) {
                cur[i] = f.base[i];
                const int64_t slot = first_slot(safe(cur[i]), f.e[i]);
                fetch_k(slot, t[i]), fetch_v(slot, t[i]);
            }
            for (bool more = true; more;) {
#pragma unroll
                for (int i = 0; i < NT; ++i) {
                    if (more && cur[i] < 0) more = false;
                    if (more) {
                        const int after = next >= 0 ? advance() : -1;      // the step after the one this buffer is refilled with
                        const int e_after = entry(safe(after));
                        const int64_t slot = first_slot(safe(next), e_next);
                        step(cur[i], t[i], [&]() __attribute__((always_inline)) { fetch_k(slot, t[i]); },
                             [&]() __attribute__((always_inline)) { fetch_v(slot, t[i]); });
                        cur[i] = next, next = after, e_next = e_after;
                    }
                }
            }
        }

        // The column's sum over its four lanes, then the four wavefronts through LDS, in wavefront order.
        const float l_col = sum_across_quarters(l);
        if (FUSED) lds_barrier();      // the previous partition's fold has read the LDS
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<f32x4*>(&s_acc[wave][c16][32 * u + 8 * i]) = f32x4{acc[0][i], acc[1][i], acc[2][i], acc[3][i]};
            *reinterpret_cast<f32x4*>(&s_acc[wave][c16][32 * u + 8 * i + 4]) = f32x4{acc[4][i], acc[5][i], acc[6][i], acc[7][i]};
        }
        if (u == 0) s_m[wave][c16] = m, s_l[wave][c16] = l_col;
        lds_barrier();
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            const int idx = tid + e * 256;
            const int cc = idx / D, d = idx % D;
            const int head_i = cc / CPH;
            const int j = j0 + cc % CPH;
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
            if constexpr (KIND == 1) A *= a.hm ? a.hm[a.hkv + kvh0 + head_i] : a.v_mult;
            if (c < count) {
                if constexpr (FUSED) {
                    // A column folds the partitions that hold its positions, as the merge does.
                    const int held = min(a.parts, (min(first + c + 1, a.max_keys) + a.piece - 1) / a.piece);
                    if (part < held) {
                        const Fold fo = fold(run_m[e], run_l[e], M, L);
                        run_a[e] = __builtin_fmaf(run_a[e], fo.keep, A * fo.take);
                        run_m[e] = fo.m, run_l[e] = fo.l;
                    }
                } else {
                    const int64_t at = ((prow + c) * a.hq + (kvh0 + head_i) * a.g + j % a.g) * a.parts + b;
                    a.po[at * D + d] = A;
                    if (d == 0) a.pm[at] = M, a.pl[at] = L;
                }
            }
        }
    }
    if constexpr (FUSED) {
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            const int idx = tid + e * 256;
            const int cc = idx / D, d = idx % D;
            const int j = j0 + cc % CPH;
            const int c = j / a.g;
            if (c < count) {
                const int head = (kvh0 + cc / CPH) * a.g + j % a.g;
                float M = run_m[e], L = run_l[e], A = run_a[e];
                if (a.sinks) {
                    const Fold fo = fold(M, L, a.sinks[head] * kLog2e, 1.0f);
                    A *= fo.keep, M = fo.m, L = fo.l;
                }
                const float o = L != 0.0f ? A / L : 0.0f;
                store_out(a.out, a.out_dtype, (int64_t)(start + c) * a.o_st + (int64_t)head * a.o_sh + d, o);
                if (a.lse && d == 0) a.lse[(int64_t)(start + c) * a.hq + head] = L != 0.0f ? __builtin_fmaf(M, kLn2, __logf(L)) : -INFINITY;
            }
        }
    }
}

// The launch: as many workgroups as the card holds at once, each taking units from the launch's counter (the caller's
// memory) until the list is exhausted. The hardware's own dispatcher binds a workgroup to an XCD by its id and starts
// workgroups strictly in order, so with units as uneven as ragged contexts make them it leaves slots idle behind a
// busy one; resident workgroups that pull the next unit themselves keep every slot busy to the end. The last workgroup
// to finish zeroes the counters for the next launch that uses them. Without counters the units are dealt in turn.
constexpr int kMfmaWaves = 2;      // wavefronts a SIMD holds (two workgroups a compute unit)
#ifndef PKV_MFMA_TILES
#define PKV_MFMA_TILES 2
#endif
constexpr int kMfmaTiles = PKV_MFMA_TILES;      // steps a wavefront keeps in flight

template <int KIND, bool F16, int HW, bool FUSED, bool MASKED>
__global__ __launch_bounds__(256, kMfmaWaves) void attend_mfma_kernel(AttendArgs a) {
    __shared__ __align__(16) float s_acc[4][kTileRows][128];
    __shared__ float s_m[4][kTileRows], s_l[4][kTileRows];
    __shared__ unsigned s_unit;
    const unsigned total = (unsigned)a.units_x * (unsigned)a.units_y;
    unsigned unit = blockIdx.x;      // the first gridDim.x units need no ticket: tickets number the units after them
    const bool pulled = a.ticket != nullptr;
    while (unit < total) {
        // (the next ticket is drawn after the unit, not during it: a returning atomic in flight makes every wait on
        // the unit's loads a wait for all of them, which costs more than the ticket's round trip)
        attend_mfma_unit<KIND, F16, HW, FUSED, MASKED, kMfmaTiles>(a, (int)(unit % (unsigned)a.units_x), (int)(unit / (unsigned)a.units_x), s_acc, s_m, s_l);
        lds_barrier();      // the unit is done with the shared arrays, and every thread has read s_unit
        if (pulled) {
            if (threadIdx.x == 0) s_unit = gridDim.x + atomicAdd(a.ticket, 1u);
            lds_barrier();
            unit = s_unit;
        } else {
            unit += gridDim.x;
        }
    }
    if (!pulled) return;
    if (threadIdx.x == 0) {
        if (atomicAdd(a.ticket + 1, 1u) == gridDim.x - 1) {
            atomicExch(a.ticket, 0u);
            atomicExch(a.ticket + 1, 0u);
        }
    }
}

}   // namespace pkv
