// Paged decode / verify-window attention for 128-wide heads: the bandwidth path of the split launch.
//
// One workgroup of 4 wavefronts per (row, KV head, query tile of QR rows, partition); a wavefront's step covers 16
// positions. Two lane layouts share the step:
//   keys    8 lanes hold one K row (two 16-byte loads each for 16-bit pages, one for 8-bit pages), so one load
//           instruction fetches 8 whole 128-byte lines; every lane dots its slice with the QR query rows
//           (v_dot2_f32_bf16 / _f16), and a transposing reduction over the 8 lanes leaves ONE finished score per
//           lane and block of four query rows: lane bits (b1 b0) = query row, (b2, b3) = which of the DPP row's four
//           positions. The softmax arithmetic (scale, mask, max, exp2, sum) therefore runs once per score, not once
//           per lane.
//   values  16 lanes (one DPP row) hold one V row, 16 bytes (8 for 8-bit pages) each; a DPP row owns four of the
//           step's positions and keeps its own online-softmax state and its own output accumulators for them.
// A wavefront serves HW adjacent KV heads at once (DPP row rho: head rho % HW, position block rho / HW), so every
// load instruction fetches HW x 128 contiguous bytes per position: 512-byte segments (2 heads of 16-bit pages, 4
// heads of 8-bit pages) are what the HBM system streams at full rate from randomly placed pages; 128-byte and
// 256-byte segments measurably are not.
// The probabilities cross from the first layout to the second through LDS as 16-bit pairs of adjacent positions,
// which is exactly the operand v_dot2 wants against the matching pairs of V values (built with v_perm_b32), so P.V
// costs one dot2 per two multiply-adds. At the end the four DPP rows and the four wavefronts are folded in a fixed
// order. No matrix cores: the kernel is bound by HBM reads of K and V.
//
// Row-exactness: position n is read by the same wavefront, DPP row and step whatever the launch; every reduction is
// a fixed balanced tree of commutative additions; masked positions contribute exact zeros; so a column's bits depend
// on its own query and keys, `piece`, `partitions` and the page kind only.
#pragma once
#include "pkv_attend_args.hpp"

namespace pkv {

// DPP controls inside a row of 16 lanes.
constexpr int kXor1 = 0xB1, kXor2 = 0x4E, kRor4 = 0x124, kRor8 = 0x128, kRor12 = 0x12C;

// The lane's partner with lane bit 2 flipped (inside its row of 16): lanes with the bit clear read lane + 4, the
// others lane - 4, by two bank-masked rotations.
PKV_DEV float dpp_xor4(float x) {
    int r = __builtin_amdgcn_update_dpp(0, (int)f2u(x), kRor12, 0xf, 0x5, false);
    r = __builtin_amdgcn_update_dpp(r, (int)f2u(x), kRor4, 0xf, 0xA, false);
    return u2f((uint32_t)r);
}

// 16-bit pairs for v_dot2: multiply-accumulate two products in FP32.
template <bool F16>
PKV_DEV float dot2(uint32_t a, uint32_t b, float c) {
    if constexpr (F16) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
    } else {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
    }
}

template <bool F16>
PKV_DEV uint32_t to16(float x) {
    if constexpr (F16) return f16_bits(x);
    return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)x);      // v_cvt_pk_bf16_f32: round to nearest even
}

// Four codes of one word as two packed BF16 pairs (codes 0,1 and 2,3), exactly.
template <int KIND>
PKV_DEV void codes4_to_bf16(uint32_t w, uint32_t& lo, uint32_t& hi) {
    if constexpr (KIND == 3) {
        const float f0 = (float)(int8_t)w, f1 = (float)(int8_t)(w >> 8), f2 = (float)(int8_t)(w >> 16), f3 = (float)(int8_t)(w >> 24);
        lo = __builtin_amdgcn_perm(f2u(f1), f2u(f0), 0x07060302);
        hi = __builtin_amdgcn_perm(f2u(f3), f2u(f2), 0x07060302);
    } else {
        lo = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)w, 1.0f, false));
        hi = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)w, 1.0f, true));
    }
}

template <int KIND>
struct Step128 {
    // keys: 16-bit pages two rows (pair A: positions base + g8, pair B: base + 8 + g8) of two 16-byte loads each;
    // 8-bit pages one 16-byte load per row. values: the DPP row's four positions.
    using VVec = typename std::conditional<KIND == 0, uint4, uint2>::type;
    uint4 k[KIND == 0 ? 4 : 2];
    VVec v[4];
    float ks, vs;      // row-scaled kinds: the scales of this lane's score position
};

// Wavefronts per SIMD the register allocation leaves room for: the keys' and values' register buffers of 16-bit pages
// are twice those of 8-bit pages, and the query slices and accumulators grow with the tile's rows; more resident
// workgroups hide each other's start-up latency, spills cost more than they give.
constexpr int attend_waves(int kind, int qr) { return qr <= 2 ? 4 : (qr <= 4 && kind != 0 ? 3 : 2); }

// Pages are a multiple of 16 positions, so the 16 positions of a step share one page table entry, which is uniform
// over the wavefront: a step's addresses are a scalar base plus per-lane offsets that do not change from step to step.
// One unit of work: (ux, uy) of a units_x x units_y list, what a workgroup of a plain launch would get as blockIdx.
// SPARSE: block lists of blocks that are a multiple of 16 positions. A tile then holds the rows of one column (the
// launcher picks QR dividing the group); the unit walks the run of the column's list, place u at position
// blocks[u / block_size] * block_size + u % block_size, cut into pieces and partitions like an ordinary row's positions;
// a step's places lie in one block and one page, so the walk stays scalar: a step of an unlisted place (id -1) or past
// the column's positions is skipped, every other step is read exactly as an ordinary row's.
template <int KIND, bool F16, int QR, int HW, bool FUSED, bool SPARSE = false>
PKV_DEV void attend128_unit(const AttendArgs& a, const int ux, const int uy) {
    static_assert(!(SPARSE && FUSED), "block lists are read by the split launch");
    constexpr int D = 128;
    constexpr int RB = (QR + 3) / 4;            // blocks of four query rows
    constexpr int EB = KIND == 0 ? 2 : 1;
    constexpr int PB = 4 / HW;                  // position blocks (of 4 positions) a wavefront's step holds
    constexpr int SPW = 4 * PB;                 // positions a wavefront's step covers
    constexpr int EPT = (QR * D + 255) / 256;
    __shared__ __align__(16) float s_acc[4][QR][D];
    __shared__ float s_m[4][QR], s_l[4][QR];
    __shared__ __align__(16) uint16_t s_p[4][4][RB * 4][4];   // [wavefront][DPP row][query row][position of the row]
    __shared__ __align__(16) float s_alpha[4][4][RB * 4];
    __shared__ __align__(16) float s_rm[4][4][RB * 4], s_rl[4][4][RB * 4];
    __shared__ int s_blocks[SPARSE ? kMaxListedBlocks : 1];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rho = lane >> 4, lam = lane & 15;
    const int b3 = (lane >> 3) & 1, b2 = (lane >> 2) & 1, b1 = (lane >> 1) & 1, b0 = lane & 1;
    const int li8 = lane & 7;
    const int q4 = 2 * b2 + b3;                 // which of the DPP row's four positions this lane's score is of
    const int hw = rho % HW, pb = rho / HW;     // the DPP row's head (of the wavefront's HW) and position block
    int bx = ux;
    const int tile = bx % a.tiles;
    bx /= a.tiles;
    const int hgroups = a.hkv / HW;
    const int kvh = (bx % hgroups) * HW + hw;   // this lane's KV head
    const int r = bx / hgroups;
    int b = uy;
    // The row's four descriptors are read together, ahead of every test that could end the unit: one memory round
    // trip instead of a chain of them at the start of every unit.
    int count_raw = *(a.counts ? a.counts + r : a.starts + r);      // (no load under a condition)
    int64_t first64 = a.firsts[r];
    int table_row = a.rows[(int64_t)r * a.rows_step];
    int start = a.starts[r];
    int off_r = *(a.offsets ? a.offsets + r : a.starts + r), off_0 = *(a.offsets ? a.offsets : a.starts);
    // (the values are taken together here, which keeps the compiler from sinking some of the loads below the tests
    // that follow, or down to the unit's end where the partials' rows are computed: one round trip, not several)
    asm volatile("" : "+v"(count_raw), "+v"(first64), "+v"(table_row), "+v"(start), "+v"(off_r), "+v"(off_0));
    // (they are the same in every lane, which the compiler cannot see through the line above: as scalars again, the
    // walk over the row's steps and its page table entries stays on the scalar unit)
    count_raw = __builtin_amdgcn_readfirstlane(count_raw), table_row = __builtin_amdgcn_readfirstlane(table_row);
    start = __builtin_amdgcn_readfirstlane(start), off_r = __builtin_amdgcn_readfirstlane(off_r), off_0 = __builtin_amdgcn_readfirstlane(off_0);
    first64 = (int64_t)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(first64 >> 32)) << 32) |
                        (uint32_t)__builtin_amdgcn_readfirstlane((int)first64));
    const int64_t prow = a.offsets ? (int64_t)(off_r - off_0) : (int64_t)r * a.columns;      // the row's first partial row
    const int count_in = a.counts ? count_raw : a.columns;
    const int64_t trow = (int64_t)table_row * a.tab_stride;
    const int count = min(count_in, a.columns);
    const int j0 = tile * QR;
    if (j0 >= count * a.g) return;
    const int c_lo = j0 / a.g;
    const int c_hi = min(count, (j0 + QR - 1) / a.g + 1);
    int64_t nk64 = first64 + c_hi;
    nk64 = nk64 < 0 ? 0 : (nk64 > (int64_t)a.max_keys ? (int64_t)a.max_keys : nk64);
    const int n_keys = (int)nk64;
    const int first = (int)(first64 < 0 ? 0 : (first64 > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : first64));
    const int n_run = SPARSE ? a.listed_keys : n_keys;      // the positions (or places of a list) the partitions divide
    const int n_pieces = (n_run + a.piece - 1) / a.piece;
    if constexpr (!FUSED) {
        // Units are taken in list order, y slowest, and a launch's tail is as long as its last units: the row's last
        // partition (usually a partial piece, the smallest unit of work) is listed after every other partition, in
        // kTailClasses rows of y by its size (a whole piece or more first, the smallest remainders last).
        const int np = min(n_pieces, a.parts);
        if (np <= 0) return;
        int cls = 0;
        if (np == n_pieces) cls = min(kTailClasses - 1, (np * a.piece - n_run) * kTailClasses / a.piece);
        if (b >= a.units_y - kTailClasses) {
            if (b - (a.units_y - kTailClasses) != cls) return;
            b = np - 1;
        } else if (b >= np - 1) {
            return;
        }
    }

    // The query row of this lane's score in each block, and the last position it sees.
    int my_lim[RB];
#pragma unroll
    for (int blk = 0; blk < RB; ++blk) {
        const int j = j0 + 4 * blk + 2 * b1 + b0;
        const int c = j / a.g;
        my_lim[blk] = (4 * blk + 2 * b1 + b0 < QR && c < count) ? first + c : -1;
    }
    // With a draft tree the window positions that row sees are those of its ancestors and itself.
    const bool tree = a.parents != nullptr || a.parents64 != nullptr;
    unsigned long long my_anc[RB];
#pragma unroll
    for (int blk = 0; blk < RB; ++blk) my_anc[blk] = (tree && my_lim[blk] >= 0) ? ancestors(a, start, my_lim[blk] - first) : 0ull;
    float k_mult = a.k_mult;
    if (KIND == 1 && a.hm) k_mult = a.hm[kvh];
    const float sscale = a.sscale * (KIND == 1 ? k_mult : 1.0f);
    const int win = a.sliding;

    // Offsets of the positions this lane reads within a step (its two K rows, its DPP row's four V rows, its score),
    // and their byte offsets from the step's first slot: the same every step but the row's last.
    const int slot_bytes = a.hkv * D * EB;
    const int koff[2] = {4 * pb + b3, 4 * pb + 2 + b3};
    const int voff[4] = {4 * pb, 4 * pb + 1, 4 * pb + 2, 4 * pb + 3};
    const int soff = 4 * pb + q4;
    const uint32_t klane = (uint32_t)(kvh * D * EB + li8 * 16);
    const uint32_t vlane = (uint32_t)(kvh * D * EB + lam * 8 * EB);
    uint32_t kvo[2], vvo[4];
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) kvo[pr] = (uint32_t)(koff[pr] * slot_bytes) + klane;
#pragma unroll
    for (int kv = 0; kv < 4; ++kv) vvo[kv] = (uint32_t)(voff[kv] * slot_bytes) + vlane;
    const uint32_t svo = (uint32_t)(soff * a.hkv + kvh);

    auto entry = [&](int base) __attribute__((always_inline)) -> int {     // the page table entry of a step (uniform over the wavefront)
        int pidx = a.page_shift >= 0 ? (base >> a.page_shift) : (base / a.page);
        pidx = pidx < a.tab_width ? pidx : a.tab_width - 1;
        return a.tables[trow + pidx];
    };
    // The step's first slot (uniform): page entry * page + base's offset in its page.
    auto first_slot = [&](int base, int e) __attribute__((always_inline)) -> int64_t {
        const int pidx = a.page_shift >= 0 ? (base >> a.page_shift) : (base / a.page);
        return (int64_t)__builtin_amdgcn_readfirstlane(e) * a.page + (base - pidx * a.page);
    };
    auto fetch_k = [&](int base, int e, Step128<KIND>& buf) __attribute__((always_inline)) {
        const int64_t slot0 = first_slot(base, e);
        const uint8_t* sbase = a.kp + slot0 * slot_bytes;
        uint32_t o[2] = {kvo[0], kvo[1]};
        uint32_t so = svo;
        if (base + SPW > n_keys) {      // the row's last step: positions past its keys read its last key instead
#pragma unroll
            for (int pr = 0; pr < 2; ++pr) o[pr] = (uint32_t)(min(koff[pr], n_keys - 1 - base) * slot_bytes) + klane;
            so = (uint32_t)(min(soff, n_keys - 1 - base) * a.hkv + kvh);
        }
#pragma unroll
        for (int pr = 0; pr < 2; ++pr) {
            if constexpr (KIND == 0) {
                buf.k[2 * pr] = *reinterpret_cast<const uint4*>(sbase + o[pr]);
                buf.k[2 * pr + 1] = *reinterpret_cast<const uint4*>(sbase + o[pr] + 128);
            } else {
                buf.k[pr] = *reinterpret_cast<const uint4*>(sbase + o[pr]);
            }
        }
        if constexpr (KIND >= 2) {
            buf.ks = (a.ks + slot0 * a.hkv)[so];
            buf.vs = (a.vs + slot0 * a.hkv)[so];
        }
    };
    auto fetch_v = [&](int base, int e, Step128<KIND>& buf) __attribute__((always_inline)) {
        const uint8_t* sbase = a.vp + first_slot(base, e) * slot_bytes;
        uint32_t o[4] = {vvo[0], vvo[1], vvo[2], vvo[3]};
        if (base + SPW > n_keys) {
#pragma unroll
            for (int kv = 0; kv < 4; ++kv) o[kv] = (uint32_t)(min(voff[kv], n_keys - 1 - base) * slot_bytes) + vlane;
        }
#pragma unroll
        for (int kv = 0; kv < 4; ++kv) {
            if constexpr (KIND == 0) buf.v[kv] = load_once16(sbase + o[kv]);
            else buf.v[kv] = load_once8(sbase + o[kv]);
        }
    };

    // A wavefront's walk over a partition's steps, and the first three steps of the unit's first partition with their
    // page table entries: those loads go out ahead of the query loads, so the keys and values wait for one memory round
    // trip after the descriptors, not for the queries' and then the entries'.
    int pi, st;
    auto start_part = [&](int part) __attribute__((always_inline)) {
        pi = part, st = wave;
        if (win > 0) {
            const int wlo = first + c_lo - win + 1;
            const int below = (wlo > 0 ? wlo : 0) / a.piece - part;
            if (below > 0) pi = part + (below + a.parts - 1) / a.parts * a.parts;
        }
    };
    if constexpr (SPARSE) {      // the tile's column's list, for the walk below (the unit's callers order the reuse)
        const int32_t* list = a.blocks + (int64_t)(start + c_lo) * a.blocks_stride;
        for (int i = tid; i < a.blocks_k; i += 256) s_blocks[i] = list[i];
        lds_barrier();
    }
    auto base_of = [&]() __attribute__((always_inline)) -> int {
        if constexpr (SPARSE) {      // the cursor's step if its block is listed and holds a position of the column, else the next such
            if (wave * SPW >= a.piece) return -1;
            for (;;) {
                if (st * SPW >= a.piece) pi += a.parts, st = wave;
                const int64_t place = (int64_t)pi * a.piece + st * SPW;
                if (place >= n_run) return -1;
                const int e = (int)div32(a.block_div, (uint32_t)place);
                const int id = __builtin_amdgcn_readfirstlane(s_blocks[e]);
                const int64_t base = (int64_t)id * a.block_size + ((int)place - e * a.block_size);
                if (id >= 0 && base < n_keys) return (int)base;
                st += 4;
            }
        } else {
            if (st * SPW >= a.piece) return -1;
            const int64_t base = (int64_t)pi * a.piece + st * SPW;
            return base < n_keys ? (int)base : -1;
        }
    };
    auto advance = [&]() __attribute__((always_inline)) -> int {
        st += 4;
        if constexpr (!SPARSE) {
            if (st * SPW >= a.piece) pi += a.parts, st = wave;
        }
        return base_of();
    };
    struct Lead {
        int base0, base1, base2, e0, e1, e2;
    };
    auto lead_of = [&](int part) __attribute__((always_inline)) -> Lead {
        Lead f;
        start_part(part);
        f.base0 = base_of();
        const int again = f.base0 >= 0 ? f.base0 : 0;      // (a wavefront without a step reads position 0's entry)
        f.e0 = entry(again);
        f.base1 = f.base0 >= 0 ? advance() : -1;
        f.e1 = entry(f.base1 >= 0 ? f.base1 : again);
        f.base2 = f.base1 >= 0 ? advance() : -1;
        f.e2 = entry(f.base2 >= 0 ? f.base2 : again);
        return f;
    };
    const int part_lo = FUSED ? 0 : b;
    const int part_hi = FUSED ? min(a.parts, n_pieces) : b + 1;
    const Lead lead_first = lead_of(part_lo);

    // The lane's slices of the tile's query rows (packed 16-bit pairs): dims 8 li8 .. +7 and 64 + 8 li8 .. +7 over
    // 16-bit pages, dims 16 li8 .. +15 over 8-bit pages (the dims its K loads cover).
    uint32_t qp[QR][8];
#pragma unroll
    for (int rr = 0; rr < QR; ++rr) {
        const int j = j0 + rr;
        const int c = j / a.g;
        uint4 w0 = make_uint4(0, 0, 0, 0), w1 = w0;
        if (c < count) {
            const uint8_t* row = a.q + ((int64_t)(start + c) * a.q_st + (int64_t)(kvh * a.g + j % a.g) * a.q_sh) * 2;
            if constexpr (KIND == 0) {
                w0 = *reinterpret_cast<const uint4*>(row + li8 * 16);
                w1 = *reinterpret_cast<const uint4*>(row + 128 + li8 * 16);
            } else {
                w0 = *reinterpret_cast<const uint4*>(row + li8 * 32);
                w1 = *reinterpret_cast<const uint4*>(row + li8 * 32 + 16);
            }
        }
        qp[rr][0] = w0.x, qp[rr][1] = w0.y, qp[rr][2] = w0.z, qp[rr][3] = w0.w;
        qp[rr][4] = w1.x, qp[rr][5] = w1.y, qp[rr][6] = w1.z, qp[rr][7] = w1.w;
    }
    float run_m[FUSED ? HW : 1][EPT], run_l[FUSED ? HW : 1][EPT], run_a[FUSED ? HW : 1][EPT];
#pragma unroll
    for (int i = 0; i < (FUSED ? HW : 1); ++i)
#pragma unroll
        for (int e = 0; e < EPT; ++e) run_m[i][e] = -INFINITY, run_l[i][e] = 0.0f, run_a[i][e] = 0.0f;

    for (int part = part_lo; part < part_hi; ++part) {
        // Per DPP row: the running maximum and sum of the query row this lane's score belongs to (per block), and the
        // row's output accumulators for the lane's 8 value dims.
        float m[RB], l[RB], acc[QR][8];
#pragma unroll
        for (int blk = 0; blk < RB; ++blk) m[blk] = -INFINITY, l[blk] = 0.0f;
#pragma unroll
        for (int rr = 0; rr < QR; ++rr)
#pragma unroll
            for (int d = 0; d < 8; ++d) acc[rr][d] = 0.0f;

        // Scores and softmax of one step: leaves the step's probabilities (pairs of adjacent positions per query row)
        // in pp and has rescaled the accumulators where a row's maximum moved.
        auto scores = [&](int base, const Step128<KIND>& buf, uint32_t (&pp)[RB * 4][2]) {
            float dpart[2][RB * 4];
#pragma unroll
            for (int pr = 0; pr < 2; ++pr) {
                uint32_t kw[8];
                if constexpr (KIND == 0) {
                    const uint4 x = buf.k[2 * pr], y = buf.k[2 * pr + 1];
                    kw[0] = x.x, kw[1] = x.y, kw[2] = x.z, kw[3] = x.w, kw[4] = y.x, kw[5] = y.y, kw[6] = y.z, kw[7] = y.w;
                } else {
                    const uint4 x = buf.k[pr];
                    codes4_to_bf16<KIND>(x.x, kw[0], kw[1]);
                    codes4_to_bf16<KIND>(x.y, kw[2], kw[3]);
                    codes4_to_bf16<KIND>(x.z, kw[4], kw[5]);
                    codes4_to_bf16<KIND>(x.w, kw[6], kw[7]);
                }
#pragma unroll
                for (int rr = 0; rr < RB * 4; ++rr) {
                    float d = 0.0f;
                    if (rr < QR) {
#pragma unroll
                        for (int j = 0; j < 8; ++j) d = dot2<F16>(qp[rr < QR ? rr : 0][j], kw[j], d);
                    }
                    dpart[pr][rr] = d;
                }
            }
            float alpha_any = 1.0f;
#pragma unroll
            for (int blk = 0; blk < RB; ++blk) {
                // transposing reduction over the 8 lanes of a K row: 8 partial sums in, 1 finished score out
                float t2[2][2];
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
#pragma unroll
                    for (int hi = 0; hi < 2; ++hi) {
                        const float x0 = dpart[pr][4 * blk + 2 * hi], x1 = dpart[pr][4 * blk + 2 * hi + 1];
                        const float keep = b0 ? x1 : x0, send = b0 ? x0 : x1;
                        t2[pr][hi] = keep + dpp<kXor1>(send);
                    }
                }
                float t1[2];
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    const float keep = b1 ? t2[pr][1] : t2[pr][0], send = b1 ? t2[pr][0] : t2[pr][1];
                    t1[pr] = keep + dpp<kXor2>(send);
                }
                const float keep = b2 ? t1[1] : t1[0], send = b2 ? t1[0] : t1[1];
                float x = keep + dpp_xor4(send);
                // the lane's score: query row 4 blk + 2 b1 + b0 at position base + soff
                const int n = base + soff;
                x *= KIND >= 2 ? sscale * buf.ks : sscale;
                bool vis = n <= my_lim[blk] && n < n_keys;
                if (tree) vis = vis && (n < first || ((my_anc[blk] >> ((n - first) & 63)) & 1ull) != 0);
                if (win > 0) vis = vis && n > my_lim[blk] - win;
                x = vis ? x : -INFINITY;
                float top = __builtin_fmaxf(x, dpp<kRor4>(x));
                top = __builtin_fmaxf(top, dpp<kRor8>(top));
                const float m_new = __builtin_fmaxf(m[blk], top);
                const float sub = m_new == -INFINITY ? 0.0f : m_new;
                const float alpha = exp2_fast(m[blk] - sub);
                const float p = exp2_fast(x - sub);
                float ps = p + dpp<kRor4>(p);
                ps = ps + dpp<kRor8>(ps);
                l[blk] = __builtin_fmaf(l[blk], alpha, ps);
                m[blk] = m_new;
                alpha_any = alpha != 1.0f ? 0.0f : alpha_any;
                s_p[wave][rho][4 * blk + 2 * b1 + b0][q4] = (uint16_t)to16<F16>(KIND >= 2 ? p * buf.vs : p);
                if (q4 == 0) s_alpha[wave][rho][4 * blk + 2 * b1 + b0] = alpha;
            }
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int h2 = 0; h2 < RB * 2; ++h2) {
                const uint4 w = *reinterpret_cast<const uint4*>(&s_p[wave][rho][2 * h2][0]);
                pp[2 * h2][0] = w.x, pp[2 * h2][1] = w.y, pp[2 * h2 + 1][0] = w.z, pp[2 * h2 + 1][1] = w.w;
            }
            if (__builtin_amdgcn_ballot_w64(alpha_any != 1.0f) != 0) {     // some row's maximum moved: rescale
#pragma unroll
                for (int blk = 0; blk < RB; ++blk) {
                    const float4 al = *reinterpret_cast<const float4*>(&s_alpha[wave][rho][4 * blk]);
                    const float av[4] = {al.x, al.y, al.z, al.w};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (4 * blk + i < QR) {
#pragma unroll
                            for (int d = 0; d < 8; ++d) acc[4 * blk + i < QR ? 4 * blk + i : 0][d] *= av[i];
                        }
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
        };
        // P.V of one step: pairs of positions (0,1) and (2,3) of the DPP row against the matching pairs of V values.
        auto values = [&](const Step128<KIND>& buf, const uint32_t (&pp)[RB * 4][2]) {
#pragma unroll
            for (int kp = 0; kp < 2; ++kp) {
                uint32_t pv[8];
                if constexpr (KIND == 0) {
                    const uint4 x = buf.v[2 * kp], y = buf.v[2 * kp + 1];
                    const uint32_t xs[4] = {x.x, x.y, x.z, x.w}, ys[4] = {y.x, y.y, y.z, y.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        pv[2 * j] = __builtin_amdgcn_perm(ys[j], xs[j], 0x05040100);
                        pv[2 * j + 1] = __builtin_amdgcn_perm(ys[j], xs[j], 0x07060302);
                    }
                } else {
                    const uint2 x = buf.v[2 * kp], y = buf.v[2 * kp + 1];
                    const uint32_t xs[2] = {x.x, x.y}, ys[2] = {y.x, y.y};
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        // bytes (x0 y0 x1 y1) and (x2 y2 x3 y3): adjacent positions' codes of one dim side by side
                        const uint32_t lo = __builtin_amdgcn_perm(ys[j], xs[j], 0x05010400);
                        const uint32_t hi = __builtin_amdgcn_perm(ys[j], xs[j], 0x07030602);
                        codes4_to_bf16<KIND>(lo, pv[4 * j], pv[4 * j + 1]);
                        codes4_to_bf16<KIND>(hi, pv[4 * j + 2], pv[4 * j + 3]);
                    }
                }
#pragma unroll
                for (int rr = 0; rr < QR; ++rr) {
#pragma unroll
                    for (int d = 0; d < 8; ++d) acc[rr][d] = dot2<F16>(pp[rr][kp], pv[d], acc[rr][d]);
                }
            }
        };

        // Software pipeline over two register buffers: a step's keys are reloaded (for two steps ahead) as soon as its
        // scores are done, its values as soon as its P.V is done, so between one and two steps are in flight; the page
        // table entries run one step further ahead. Every load of the loop is issued unconditionally (past the
        // wavefront's last step it re-reads its first step, which the caches hold): with straight-line loads the
        // compiler counts the outstanding ones exactly and waits only for the step it is about to use.
        Step128<KIND> bufA, bufB;
        uint32_t pp[RB * 4][2];
        const Lead f = part == part_lo ? lead_first : lead_of(part);
        int base0 = f.base0, base1 = f.base1, base2 = f.base2;
        if (base0 >= 0) {
            const int again = base0;
            auto safe = [&](int base) __attribute__((always_inline)) { return base >= 0 ? base : again; };
            const int e0 = f.e0, e1 = f.e1;
            int e2 = f.e2;
            fetch_k(base0, e0, bufA), fetch_v(base0, e0, bufA);
            fetch_k(safe(base1), e1, bufB), fetch_v(safe(base1), e1, bufB);
            for (;;) {
                const int base3 = base2 >= 0 ? advance() : -1;
                const int e3 = entry(safe(base3));
                scores(base0, bufA, pp);
                fetch_k(safe(base2), e2, bufA);
                values(bufA, pp);
                fetch_v(safe(base2), e2, bufA);
                if (base1 < 0) break;
                const int base4 = base3 >= 0 ? advance() : -1;
                const int e4 = entry(safe(base4));
                scores(base1, bufB, pp);
                fetch_k(safe(base3), e3, bufB);
                values(bufB, pp);
                fetch_v(safe(base3), e3, bufB);
                if (base2 < 0) break;
                base0 = base2, base1 = base3, base2 = base4, e2 = e4;
            }
        }

        // Fold the DPP rows that served the same head (its position blocks): every lane needs each query row's
        // maximum and sum of those rows.
#pragma unroll
        for (int blk = 0; blk < RB; ++blk) {
            if (q4 == 0) s_rm[wave][rho][4 * blk + 2 * b1 + b0] = m[blk], s_rl[wave][rho][4 * blk + 2 * b1 + b0] = l[blk];
        }
        __builtin_amdgcn_wave_barrier();
        float wm[QR], wl[QR];
#pragma unroll
        for (int rr = 0; rr < QR; ++rr) {
            float top = s_rm[wave][hw][rr];
#pragma unroll
            for (int o = 1; o < PB; ++o) top = __builtin_fmaxf(top, s_rm[wave][hw + HW * o][rr]);
            const float sub = top == -INFINITY ? 0.0f : top;
            float lsum = 0.0f;
#pragma unroll
            for (int o = 0; o < PB; ++o) lsum = __builtin_fmaf(s_rl[wave][hw + HW * o][rr], exp2_fast(s_rm[wave][hw + HW * o][rr] - sub), lsum);
            if constexpr (PB > 1) {
                const float w = exp2_fast(s_rm[wave][rho][rr] - sub);
#pragma unroll
                for (int d = 0; d < 8; ++d) acc[rr][d] = sum_over_groups<16 * HW>(acc[rr][d] * w);
            }
            wm[rr] = top, wl[rr] = lsum;
        }
        // Then the four wavefronts, one head of the wavefront at a time through LDS, in wavefront order.
#pragma unroll
        for (int head_i = 0; head_i < HW; ++head_i) {
            if (FUSED || head_i > 0) lds_barrier();      // the previous fold has read the LDS
            if (rho == head_i) {
#pragma unroll
                for (int rr = 0; rr < QR; ++rr) {
                    *reinterpret_cast<float4*>(&s_acc[wave][rr][lam * 8]) = make_float4(acc[rr][0], acc[rr][1], acc[rr][2], acc[rr][3]);
                    *reinterpret_cast<float4*>(&s_acc[wave][rr][lam * 8 + 4]) = make_float4(acc[rr][4], acc[rr][5], acc[rr][6], acc[rr][7]);
                    if (lam == 0) s_m[wave][rr] = wm[rr], s_l[wave][rr] = wl[rr];
                }
            }
            lds_barrier();
            const int head_kv = (kvh - hw) + head_i;      // the KV head being folded (uniform)
            float vm = a.v_mult;
            if (KIND == 1 && a.hm) vm = a.hm[a.hkv + head_kv];
            if (KIND != 1) vm = 1.0f;
#pragma unroll
            for (int e = 0; e < EPT; ++e) {
                const int idx = tid + e * 256;
                if (idx < QR * D) {
                    const int rr = idx / D, d = idx % D;
                    float M = s_m[0][rr];
#pragma unroll
                    for (int w = 1; w < 4; ++w) M = __builtin_fmaxf(M, s_m[w][rr]);
                    const float sub = M == -INFINITY ? 0.0f : M;
                    float L = 0.0f, A = 0.0f;
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const float f = exp2_fast(s_m[w][rr] - sub);
                        L = __builtin_fmaf(s_l[w][rr], f, L);
                        A = __builtin_fmaf(s_acc[w][rr][d], f, A);
                    }
                    A *= vm;
                    const int j = j0 + rr;
                    const int c = j / a.g;
                    if (c < count) {
                        if constexpr (FUSED) {
                            const int held = min(a.parts, (min(first + c + 1, a.max_keys) + a.piece - 1) / a.piece);
                            if (part < held) {
                                const Fold f = fold(run_m[head_i][e], run_l[head_i][e], M, L);
                                run_a[head_i][e] = __builtin_fmaf(run_a[head_i][e], f.keep, A * f.take);
                                run_m[head_i][e] = f.m, run_l[head_i][e] = f.l;
                            }
                        } else {
                            const int64_t at = ((prow + c) * a.hq + head_kv * a.g + j % a.g) * a.parts + b;
                            a.po[at * D + d] = A;
                            if (d == 0) a.pm[at] = M, a.pl[at] = L;
                        }
                    }
                }
            }
        }
    }
    if constexpr (FUSED) {
#pragma unroll
        for (int head_i = 0; head_i < HW; ++head_i) {
            const int head_kv = (kvh - hw) + head_i;
#pragma unroll
            for (int e = 0; e < EPT; ++e) {
                const int idx = tid + e * 256;
                if (idx < QR * D) {
                    const int rr = idx / D, d = idx % D;
                    const int j = j0 + rr;
                    const int c = j / a.g;
                    if (c < count) {
                        const int head = head_kv * a.g + j % a.g;
                        float M = run_m[head_i][e], L = run_l[head_i][e], A = run_a[head_i][e];
                        if (a.sinks) {
                            const Fold f = fold(M, L, a.sinks[head] * kLog2e, 1.0f);
                            A *= f.keep, M = f.m, L = f.l;
                        }
                        const float o = L != 0.0f ? A / L : 0.0f;
                        store_out(a.out, a.out_dtype, (int64_t)(start + c) * a.o_st + (int64_t)head * a.o_sh + d, o);
                        if (a.lse && d == 0) {
                            a.lse[(int64_t)(start + c) * a.hq + head] = L != 0.0f ? __builtin_fmaf(M, kLn2, __logf(L)) : -INFINITY;
                        }
                    }
                }
            }
        }
    }
}

// The launch: as many workgroups as the card holds at once, each taking units from the launch's counter (the caller's
// memory) until the list is exhausted. The hardware's own dispatcher binds a workgroup to an XCD by its id and starts
// workgroups strictly in order, so with units as uneven as ragged contexts make them it leaves slots idle behind a
// busy one; resident workgroups that pull the next unit themselves keep every slot busy to the end. The last workgroup
// to finish zeroes the counters for the next launch that uses them. Without counters the units are dealt in turn.
template <int KIND, bool F16, int QR, int HW, bool FUSED, bool SPARSE = false>
__global__ __launch_bounds__(256, attend_waves(KIND, QR)) void attend128_kernel(AttendArgs a) {
    __shared__ unsigned s_unit;
    const unsigned total = (unsigned)a.units_x * (unsigned)a.units_y;
    unsigned u = blockIdx.x;      // the first gridDim.x units need no ticket: tickets number the units after them
    const bool pulled = a.ticket != nullptr;
    while (u < total) {
        // (the next ticket is drawn after the unit, not during it: a returning atomic in flight makes every wait on
        // the unit's loads a wait for all of them, which costs more than the ticket's round trip)
        attend128_unit<KIND, F16, QR, HW, FUSED, SPARSE>(a, (int)(u % (unsigned)a.units_x), (int)(u / (unsigned)a.units_x));
        lds_barrier();      // the unit is done with the shared arrays, and every thread has read s_unit
        if (pulled) {
            if (threadIdx.x == 0) s_unit = gridDim.x + atomicAdd(a.ticket, 1u);
            lds_barrier();
            u = s_unit;
        } else {
            u += gridDim.x;
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
