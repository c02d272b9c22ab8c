// Latent attention (multi-head latent attention, absorbed) over a paged cache of compressed rows, for gfx950: decode
// tokens and verify windows of every query head over rows that hold a position's latent (rank R) and then its rotary
// key (width P); the latent is the position's value too. What the reference's latent-attention kernels module computes
// (kernels/techniques/attention/latent-attention/torch-ext/latent_attention/__init__.py:153-229, _kernels.py), split
// over KV partitions and merged in partition order.
//
// A workgroup of four wavefronts serves one unit: 16 query rows (a batch row's columns times its heads, flattened
// column-major) over pieces b, b + parts, ... of the row's positions, 32 positions a step. The step's cache rows go
// through LDS once ([position][value], 16-bit) and feed both products on the matrix pipe:
//   S^T = K Q^T   v_mfma_f32_16x16x32: A = cache rows as they lie (a lane: one position, 8 adjacent values), B = the
//                 query tile. The (R + P) / 32 k-steps are dealt to the four wavefronts (each keeps its k-steps of the
//                 queries in registers for the unit), whose partial tiles are added through LDS in a fixed order, so
//                 every wavefront holds the same scores.
//   O^T += V^T P^T  v_mfma_f32_16x16x32: B = the probabilities straight from the score tiles' registers (the D layout
//                 of two 16-position tiles is the B layout of one 32-position k-step, k-slot e of quarter g being
//                 position 4 g + e of tile 0 for e < 4, of tile 1 else); A = V^T read from the same LDS rows by
//                 ds_read_b64_tr_b16, which hands a lane 4 consecutive positions of one value. Each wavefront owns R / 4
//                 of the output values.
// The online softmax runs in base 2 on scores times scale * log2(e). A query row's bits depend on its own query and
// positions, `piece` and `partitions` only: the matrix pipe computes each output element from its own row and column,
// positions past a row's own contribute exact zeros, every sum has a fixed order.
//
// Arithmetic intensity: one position is (R + P) * e bytes and 2 * (2 R + P) * rows flops; at 16 heads a launch is
// HBM-bound, at 128 heads (8 tiles a row) the tiles of one (row, partition) are placed on one XCD so that its L2 serves
// the cache rows to all of them.
#include "pkv_attend_mfma.hpp"
#include "pkv_launch.hpp"

namespace pkv {
namespace {

typedef short s16x4 __attribute__((ext_vector_type(4)));

struct LatentArgs {
    const uint8_t* q;
    const uint8_t* cache;
    const float* scales;
    const int32_t* tables;
    const int32_t* rows;
    int rows_step;
    const int32_t* starts;
    const int32_t* counts;
    const int64_t* firsts;
    float* po;
    float* pm;
    float* pl;
    void* out;
    float* lse;
    const float* sinks;
    int64_t q_st, q_sh, o_st, o_sh, tab_stride, pairs;
    int tab_width, n_rows, columns, heads, page, parts, gy, piece, tiles, max_keys, scales_per_row, out_dtype;
    Div32 page_div;
    float sscale;
};

// 4 consecutive positions (rows of the LDS tile) of one value, transposed on the way out of LDS: lane 4 j + c of a
// 16-lane group points at row j's values 4 c .. 4 c + 3; lane i of the group receives value i of rows 0 .. 3.
PKV_DEV u32x2 lds_transposed(const uint8_t* p) {
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p));
    return __builtin_bit_cast(u32x2, v);
}

// NT: query tiles (of 16 rows) a workgroup serves over one staging of the cache rows: 1 where a row's columns times
// heads fit one tile, else 2 (each tile is then two wavefronts' work: the staging, the barriers and half of the softmax
// are shared by twice the rows). A tile's score is the sum of four chains of k-steps (chain c: k-steps c, c + 4, ...)
// added as ((0 + 1) + 2) + 3 whichever wavefront computed them, so a row's bits do not depend on NT.
template <int R, int P, bool F16, bool FP8, int NT>
__global__ __launch_bounds__(256, NT == 1 ? 3 : 2) void latent_kernel(LatentArgs a) {
    constexpr int W = R + P;                   // values a cache row holds
    constexpr int ROWB = W * 2 + 32;           // bytes between rows in LDS: 32 mod 64 words apart, so that 16 rows' 32-byte
                                               // reads fall on different banks
    constexpr int KS = W / 32, KSL = R / 32;   // k-steps of the scores; the first KSL are the latent's
    constexpr int WPT = 4 / NT;                // wavefronts a query tile
    constexpr int FT = (R / 16) / WPT;         // 16-value output tiles a wavefront owns
    constexpr int EB = FP8 ? 1 : 2;
    constexpr int CPR = W * EB / 16;           // 16-byte chunks of a cache row
    constexpr int NL = (CPR + 7) / 8;          // chunks a thread moves a step
    constexpr int KPC = (KS + 3) / 4;          // k-steps a chain holds
    constexpr int NPART = FP8 ? 16 : 8;        // floats a lane's partial score tiles take (latent and rotary apart for E4M3)
    __shared__ __align__(16) uint8_t s_k[32 * ROWB];
    __shared__ float s_part[NT][4][NPART][64];
    __shared__ float s_scale[FP8 ? 32 : 1][2];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, g = lane >> 4, li = lane & 15;
    const int wt = wave / WPT, sub = wave % WPT;      // the wavefront's tile of the workgroup's, and its place among that tile's
    // Workgroups go to the XCDs in turn: the tile groups of one (row, partition) take consecutive places of one XCD.
    const int64_t bid = blockIdx.x;
    const int64_t place = bid >> 3;
    const int64_t pair = (place / a.tiles) * 8 + (bid & 7);
    const int group = (int)(place % a.tiles);
    if (pair >= a.pairs) return;
    const int r = (int)(pair / a.gy), b = (int)(pair % a.gy);
    int count = a.columns;
    if (a.counts) count = min(a.counts[r], a.columns);
    const int H = a.heads;
    const int live_rows = count * H;
    if (group * NT * 16 >= live_rows) return;
    const int64_t first64 = a.firsts[r];
    const int first = (int)(first64 < 0 ? 0 : (first64 > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : first64));
    const int c_hi = (min((group + 1) * NT * 16, live_rows) - 1) / H + 1;      // columns the group's rows reach
    const int n_keys = min(first + c_hi, a.max_keys);
    const int n_pieces = (n_keys + a.piece - 1) / a.piece;
    if (b >= n_pieces) return;
    const int64_t trow = (int64_t)a.rows[(int64_t)r * a.rows_step] * a.tab_stride;
    const int start = a.starts[r];

    // The lane's query row (column li of its wavefront's score tiles).
    const int j0 = (group * NT + wt) * 16;
    const int jq = j0 + li, colq = jq / H, headq = jq - colq * H;
    const bool liveq = colq < count;
    const int lim = liveq ? first + colq : -1;
    const int unmasked = min(first + j0 / H + 1, n_keys);      // positions below it are seen by every live row of the tile

    // The wavefront's chains of the lane's query row, as the matrix pipe takes them (a dead row: zeros).
    u32x4 bq[NT][KPC];
#pragma unroll
    for (int c = 0; c < NT; ++c) {
#pragma unroll
        for (int k4 = 0; k4 < KPC; ++k4) {
            const int ks = k4 * 4 + sub + c * WPT;
            bq[c][k4] = u32x4{0u, 0u, 0u, 0u};
            if (liveq && ks < KS)
                bq[c][k4] = *reinterpret_cast<const u32x4*>(a.q + ((int64_t)(start + colq) * a.q_st + (int64_t)headq * a.q_sh) * 2 + ks * 64 + g * 16);
        }
    }

    // A step's cache rows: eight threads move one row (thread t: row t / 8, its 16-byte chunks t % 8, t % 8 + 8, ...), so
    // a thread looks up one slot a step. The page table entry is read a step ahead of the row itself, which is read a
    // step ahead of its use: no load waits for another inside a step.
    const int my_row = tid >> 3, my_ch = tid & 7;
    u32x4 held[NL];
    int entry = 0;
    float held_scale[2] = {1.0f, 1.0f};
    auto fetch_entry = [&](int base) __attribute__((always_inline)) {
        int n = base + my_row;
        n = n < n_keys ? n : n_keys - 1;
        const int pidx = (int)div32(a.page_div, (uint32_t)n);
        entry = a.tables[trow + (pidx < a.tab_width ? pidx : a.tab_width - 1)];
    };
    auto fetch = [&](int base) __attribute__((always_inline)) {
        int n = base + my_row;
        n = n < n_keys ? n : n_keys - 1;
        const int64_t slot = (int64_t)entry * a.page + (n - (int)div32(a.page_div, (uint32_t)n) * a.page);
        const uint8_t* row = a.cache + slot * (W * EB) + my_ch * 16;
#pragma unroll
        for (int l = 0; l < NL; ++l)
            if (CPR % 8 == 0 || my_ch + 8 * l < CPR) held[l] = *reinterpret_cast<const u32x4*>(row + l * 128);
        if constexpr (FP8) {
            if (my_ch == 0) {
                const float* sc = a.scales + slot * a.scales_per_row;
                held_scale[0] = sc[0];
                held_scale[1] = a.scales_per_row > 1 ? sc[1] : sc[0];
            }
        }
    };
    auto stage = [&]() __attribute__((always_inline)) {
        uint8_t* row = s_k + my_row * ROWB + my_ch * (FP8 ? 32 : 16);
#pragma unroll
        for (int l = 0; l < NL; ++l) {
            if (CPR % 8 == 0 || my_ch + 8 * l < CPR) {
                if constexpr (FP8) {      // 16 codes: 16 values of the queries' type, exactly
                    const uint32_t w[4] = {held[l].x, held[l].y, held[l].z, held[l].w};
                    uint32_t o[8];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const f32x2 lo = e4m3_pair<false>(w[k]), hi = e4m3_pair<true>(w[k]);
                        o[2 * k] = pair16<F16>(lo.x, lo.y), o[2 * k + 1] = pair16<F16>(hi.x, hi.y);
                    }
                    u32x4* at = reinterpret_cast<u32x4*>(row + l * 256);
                    at[0] = u32x4{o[0], o[1], o[2], o[3]};
                    at[1] = u32x4{o[4], o[5], o[6], o[7]};
                } else {
                    *reinterpret_cast<u32x4*>(row + l * 128) = held[l];
                }
            }
        }
        if constexpr (FP8) {
            if (my_ch == 0) s_scale[my_row][0] = held_scale[0], s_scale[my_row][1] = held_scale[1];
        }
    };

    // The workgroup's steps: steps 0 .. of pieces b, b + parts, ...
    const int steps_per_piece = a.piece / 32;
    int pi = b, st = 0;
    auto base_of = [&]() __attribute__((always_inline)) -> int {
        const int64_t base = (int64_t)pi * a.piece + st * 32;
        return base < n_keys ? (int)base : -1;
    };
    auto advance = [&]() __attribute__((always_inline)) -> int {
        if (++st >= steps_per_piece) pi += a.parts, st = 0;
        return base_of();
    };

    float m = -INFINITY, l = 0.0f;
    f32x4 acc[FT];
#pragma unroll
    for (int t = 0; t < FT; ++t) acc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    int base = base_of();      // (>= 0: b < n_pieces)
    fetch_entry(base);
    fetch(base);
    int next = advance();
    if (next >= 0) fetch_entry(next);
    while (base >= 0) {
        stage();
        lds_barrier();
        int after = -1;
        if (next >= 0) {
            fetch(next);
            after = advance();
            if (after >= 0) fetch_entry(after);
        }
        // -- the step's scores: this wavefront's chains of its tile, both 16-position halves of the step. The operands are
        // read from LDS a few products ahead (a ring), so a read's latency is not waited for before every product. A
        // chain's k-step past the last (the wavefronts do not all have as many) multiplies the last one's rows by the
        // zeros its queries hold there.
        const uint8_t* krow = s_k + li * ROWB + g * 16;
        {
            constexpr int NOPS = NT * KPC;
            constexpr int RING = NOPS < 4 ? NOPS : 4;
            u32x4 ka[RING][2];
            f32x4 sl[NT][2], sr[NT][2];
#pragma unroll
            for (int c = 0; c < NT; ++c)
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) sl[c][hh] = f32x4{0.0f, 0.0f, 0.0f, 0.0f}, sr[c][hh] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            auto read_k = [&](auto ic) __attribute__((always_inline)) {
                constexpr int i = decltype(ic)::value;
                constexpr int c = i / KPC, k4 = i % KPC;
                int ks = k4 * 4 + sub + c * WPT;
                ks = ks < KS ? ks : KS - 1;
                ka[i % RING][0] = *reinterpret_cast<const u32x4*>(krow + ks * 64);
                ka[i % RING][1] = *reinterpret_cast<const u32x4*>(krow + 16 * ROWB + ks * 64);
            };
            static_for<RING - 1>([&](auto ic) __attribute__((always_inline)) { read_k(ic); });
            static_for<NOPS>([&](auto ic) __attribute__((always_inline)) {
                constexpr int i = decltype(ic)::value;
                constexpr int c = i / KPC, k4 = i % KPC;
                if constexpr (i + RING - 1 < NOPS) read_k(std::integral_constant<int, i + RING - 1>{});
                // (k-steps from KSL on are the rotary key's: a chain's k4 decides where the latent's k-steps come in fours)
                const bool rotary = FP8 && (KSL % 4 == 0 ? k4 * 4 >= KSL : k4 * 4 + sub + c * WPT >= KSL);
                if (rotary) {
                    sr[c][0] = mfma_k32<F16>(ka[i % RING][0], bq[c][k4], sr[c][0]);
                    sr[c][1] = mfma_k32<F16>(ka[i % RING][1], bq[c][k4], sr[c][1]);
                } else {
                    sl[c][0] = mfma_k32<F16>(ka[i % RING][0], bq[c][k4], sl[c][0]);
                    sl[c][1] = mfma_k32<F16>(ka[i % RING][1], bq[c][k4], sl[c][1]);
                }
            });
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * (RING - 1), 0);
            static_for<NOPS>([&](auto) __attribute__((always_inline)) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            });
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int c = 0; c < NT; ++c) {
                float (&mine)[NPART][64] = s_part[wt][sub + c * WPT];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    mine[i][lane] = sl[c][0][i], mine[4 + i][lane] = sl[c][1][i];
                    if constexpr (FP8) mine[8 + i][lane] = sr[c][0][i], mine[12 + i][lane] = sr[c][1][i];
                }
            }
        }
        lds_barrier();
        float x[8];
        const bool masked = base + 32 > unmasked;      // (the same for the whole wavefront)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float latent = ((s_part[wt][0][e][lane] + s_part[wt][1][e][lane]) + s_part[wt][2][e][lane]) + s_part[wt][3][e][lane];
            const int at = (e >> 2) * 16 + 4 * g + (e & 3);      // the value's position in the step
            float v = latent;
            if constexpr (FP8) {
                const float rotary = ((s_part[wt][0][8 + e][lane] + s_part[wt][1][8 + e][lane]) + s_part[wt][2][8 + e][lane]) + s_part[wt][3][8 + e][lane];
                v = __builtin_fmaf(latent, s_scale[at][0], rotary * s_scale[at][1]);
            }
            x[e] = v * a.sscale;
            if (masked) {
                const int n = base + at;
                x[e] = (n <= lim && n < n_keys) ? x[e] : -INFINITY;
            }
        }
        float top = __builtin_fmaxf(__builtin_fmaxf(__builtin_fmaxf(x[0], x[1]), __builtin_fmaxf(x[2], x[3])),
                                    __builtin_fmaxf(__builtin_fmaxf(x[4], x[5]), __builtin_fmaxf(x[6], x[7])));
        top = max_across_quarters(top);
        const float m_new = __builtin_fmaxf(m, top);
        const float sub2 = m_new == -INFINITY ? 0.0f : m_new;
        const float alpha = exp2_fast(m - sub2);
        float p[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) p[e] = exp2_fast(x[e] - sub2);
        const float sum = sum_across_quarters(((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7])));
        l = __builtin_fmaf(l, alpha, sum);
        m = m_new;
        if constexpr (FP8) {      // a value is its code times its position's latent scale: the scale rides on the probability
#pragma unroll
            for (int e = 0; e < 8; ++e) p[e] *= s_scale[(e >> 2) * 16 + 4 * g + (e & 3)][0];
        }
        const u32x4 bp = {pair16<F16>(p[0], p[1]), pair16<F16>(p[2], p[3]), pair16<F16>(p[4], p[5]), pair16<F16>(p[6], p[7])};
        // -- the wavefront's share of the values (the accumulators move only when some row's maximum did: x 1 is exact)
        const bool rescale = __ballot(alpha != 1.0f) != 0ull;
        const uint8_t* vrow = s_k + (4 * g + (li >> 2)) * ROWB + (li & 3) * 8 + sub * FT * 32;
        if (rescale) {
#pragma unroll
            for (int t = 0; t < FT; ++t) acc[t] *= alpha;
        }
        {
            constexpr int VR = FT < 5 ? FT : 5;      // value operands read ahead, as the keys' are
            u32x2 va[VR][2];
            auto read_v = [&](auto ic) __attribute__((always_inline)) {
                constexpr int t = decltype(ic)::value;
                va[t % VR][0] = lds_transposed(vrow + t * 32);
                va[t % VR][1] = lds_transposed(vrow + 16 * ROWB + t * 32);
            };
            static_for<VR - 1>([&](auto ic) __attribute__((always_inline)) { read_v(ic); });
            static_for<FT>([&](auto ic) __attribute__((always_inline)) {
                constexpr int t = decltype(ic)::value;
                if constexpr (t + VR - 1 < FT) read_v(std::integral_constant<int, t + VR - 1>{});
                acc[t] = mfma_k32<F16>(u32x4{va[t % VR][0].x, va[t % VR][0].y, va[t % VR][1].x, va[t % VR][1].y}, bp, acc[t]);
            });
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * (VR - 1), 0);
            static_for<FT>([&](auto) __attribute__((always_inline)) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            });
            __builtin_amdgcn_sched_barrier(0);
        }
        lds_barrier();      // (the barriers order LDS only: the next step's loads stay in flight across them)
        base = next, next = after;
    }
    if (!liveq) return;
    const int64_t index = ((int64_t)((int64_t)r * a.columns + colq) * H + headq) * a.parts + b;
#pragma unroll
    for (int t = 0; t < FT; ++t)
        *reinterpret_cast<f32x4*>(a.po + index * R + (sub * FT + t) * 16 + 4 * g) = acc[t];
    if (sub == 0 && g == 0) a.pm[index] = m, a.pl[index] = l;
}

// One workgroup of 64 threads a (batch row, column, head): the partitions' states folded in partition order, the sink
// last; R / 64 values a thread.
template <int R>
__global__ __launch_bounds__(64) void latent_merge_kernel(LatentArgs a) {
    const int prow = blockIdx.x, head = blockIdx.y;
    const int r = prow / a.columns, col = prow - r * a.columns;
    int count = a.columns;
    if (a.counts) count = min(a.counts[r], a.columns);
    if (col >= count) return;
    const int64_t first64 = a.firsts[r];
    const int first = (int)(first64 < 0 ? 0 : (first64 > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : first64));
    const int n_keys = min(first + col + 1, a.max_keys);
    const int n_pieces = (n_keys + a.piece - 1) / a.piece;
    const int np = min(a.parts, n_pieces);
    const int64_t index = ((int64_t)prow * a.heads + head) * a.parts;
    float M = -INFINITY, L = 0.0f, acc[R / 64];
#pragma unroll
    for (int i = 0; i < R / 64; ++i) acc[i] = 0.0f;
    // Four partitions' states are requested together (past the last one the last again, so every load is issued) and
    // folded one by one in partition order: a fold waits for its own state only once in four.
    constexpr int AHEAD = 4;
    for (int b0 = 0; b0 < np; b0 += AHEAD) {
        float pm[AHEAD], pl[AHEAD], po[AHEAD][R / 64];
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) {
            const int64_t at = index + min(b0 + j, np - 1);
            pm[j] = a.pm[at], pl[j] = a.pl[at];
#pragma unroll
            for (int i = 0; i < R / 64; ++i) po[j][i] = a.po[at * R + i * 64 + threadIdx.x];
        }
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) {
            if (b0 + j < np) {
                const Fold f = fold(M, L, pm[j], pl[j]);
#pragma unroll
                for (int i = 0; i < R / 64; ++i) acc[i] = __builtin_fmaf(acc[i], f.keep, po[j][i] * f.take);
                M = f.m, L = f.l;
            }
        }
    }
    if (a.sinks) {      // one more position with no value
        const float sink = a.sinks[head] * kLog2e;
        const float top = __builtin_fmaxf(M, sink);
        const float sub = top == -INFINITY ? 0.0f : top;
        const float keep = exp2_fast(M - sub);
        L = __builtin_fmaf(L, keep, exp2_fast(sink - sub));
#pragma unroll
        for (int i = 0; i < R / 64; ++i) acc[i] *= keep;
        M = top;
    }
    const int64_t token = (int64_t)a.starts[r] + col;
    const float inv = L > 0.0f ? 1.0f / L : 0.0f;
#pragma unroll
    for (int i = 0; i < R / 64; ++i)
        store_out(a.out, a.out_dtype, token * a.o_st + (int64_t)head * a.o_sh + i * 64 + threadIdx.x, acc[i] * inv);
    // (a NaN sum, from a NaN query, stays a NaN: a fault upstream shows in the log-sum-exp as it does in the output)
    if (a.lse && threadIdx.x == 0) a.lse[token * a.heads + head] = (L > 0.0f || L != L) ? (M + __builtin_log2f(L)) * kLn2 : -INFINITY;
}

template <int R, int P, int NT>
int launch_tiles(const LatentArgs& a, bool f16, bool fp8, hipStream_t stream) {
    const int64_t blocks = (a.pairs + 7) / 8 * 8 * a.tiles;
    if (blocks > 0x7fffffff) return CRIT_PKV_E_GEOMETRY;
    const dim3 grid((unsigned)blocks);
    if (fp8) {
        if (f16) hipLaunchKernelGGL((latent_kernel<R, P, true, true, NT>), grid, dim3(256), 0, stream, a);
        else hipLaunchKernelGGL((latent_kernel<R, P, false, true, NT>), grid, dim3(256), 0, stream, a);
    } else {
        if (f16) hipLaunchKernelGGL((latent_kernel<R, P, true, false, NT>), grid, dim3(256), 0, stream, a);
        else hipLaunchKernelGGL((latent_kernel<R, P, false, false, NT>), grid, dim3(256), 0, stream, a);
    }
    return hip_code(hipGetLastError());
}

template <int R, int P>
int launch_shape(const LatentArgs& a, bool f16, bool fp8, int phases, hipStream_t stream) {
    if (phases != 2) {
        // (a launch whose rows fit one tile each takes the one-tile workgroups: three a compute unit)
        LatentArgs u = a;
        const int tiles = (a.columns * a.heads + 15) / 16;
        u.tiles = tiles > 1 ? (tiles + 1) / 2 : 1;
        const int bad = tiles > 1 ? launch_tiles<R, P, 2>(u, f16, fp8, stream) : launch_tiles<R, P, 1>(u, f16, fp8, stream);
        if (bad) return bad;
    }
    if (phases != 1) {
        hipLaunchKernelGGL((latent_merge_kernel<R>), dim3((unsigned)(a.n_rows * a.columns), (unsigned)a.heads), dim3(64), 0, stream, a);
        return hip_code(hipGetLastError());
    }
    return 0;
}

}   // namespace

int launch_latent(const crit_pkv_latent_params* p, hipStream_t stream) {
    if (!p || !p->q || !p->cache || !p->tables || !p->rows || !p->starts || !p->firsts || !p->out || !p->partial_out ||
        !p->partial_max || !p->partial_sum)
        return CRIT_PKV_E_NULL;
    const bool fp8 = p->cache_dtype == 2;
    if (p->cache_dtype < 0 || p->cache_dtype > 2 || (p->q_dtype != CRIT_PKV_BF16 && p->q_dtype != CRIT_PKV_F16)) return CRIT_PKV_E_DTYPE;
    if (!fp8 && p->cache_dtype != (p->q_dtype == CRIT_PKV_F16 ? 1 : 0)) return CRIT_PKV_E_DTYPE;      // 16-bit rows in the queries' type
    if (fp8 && (!p->scales || (p->scales_per_row != 1 && p->scales_per_row != 2))) return CRIT_PKV_E_NULL;
    if (p->out_dtype != CRIT_PKV_F32 && p->out_dtype != CRIT_PKV_BF16 && p->out_dtype != CRIT_PKV_F16) return CRIT_PKV_E_DTYPE;
    if (p->n_rows < 1 || p->columns < 1 || p->columns > CRIT_PKV_MAX_COLUMNS || p->heads < 1 || p->page < 1 || p->table_width < 1 ||
        (int64_t)p->n_rows * p->columns > 0x7fffffff || p->heads > 65535)
        return CRIT_PKV_E_GEOMETRY;
    if (p->q_stride_t % 8 || p->q_stride_h % 8 || (reinterpret_cast<uintptr_t>(p->q) % 16) || (reinterpret_cast<uintptr_t>(p->cache) % 16))
        return CRIT_PKV_E_GEOMETRY;
    if (p->partitions < 1 || p->partitions > 65535 || p->piece < 32 || p->piece % 32) return CRIT_PKV_E_WORKSPACE;
    LatentArgs a;
    a.q = reinterpret_cast<const uint8_t*>(p->q), a.cache = reinterpret_cast<const uint8_t*>(p->cache), a.scales = p->scales;
    a.tables = p->tables, a.rows = reinterpret_cast<const int32_t*>(p->rows), a.rows_step = p->rows_are_64 ? 2 : 1;
    a.starts = p->starts, a.counts = p->counts, a.firsts = p->firsts;
    a.po = p->partial_out, a.pm = p->partial_max, a.pl = p->partial_sum;
    a.out = p->out, a.lse = p->lse, a.sinks = p->sinks;
    a.q_st = p->q_stride_t, a.q_sh = p->q_stride_h, a.o_st = p->out_stride_t, a.o_sh = p->out_stride_h, a.tab_stride = p->table_stride;
    a.tab_width = p->table_width, a.n_rows = p->n_rows, a.columns = p->columns, a.heads = p->heads, a.page = p->page;
    a.page_div = make_div32((uint32_t)p->page);
    a.parts = p->partitions, a.piece = p->piece, a.scales_per_row = p->scales_per_row, a.out_dtype = p->out_dtype;
    a.sscale = p->scale * kLog2e;
    a.tiles = (p->columns * p->heads + 15) / 16;
    const int64_t table_keys = (int64_t)p->table_width * p->page;
    a.max_keys = (int)(table_keys < 0x3fffffff ? table_keys : 0x3fffffff);
    if ((int64_t)p->partitions * p->piece > 0x3fffffff) return CRIT_PKV_E_WORKSPACE;
    const int64_t live_parts = ((int64_t)a.max_keys + p->piece - 1) / p->piece;
    a.gy = (int)(live_parts < p->partitions ? live_parts : p->partitions);
    a.pairs = (int64_t)p->n_rows * a.gy;
    const bool f16 = p->q_dtype == CRIT_PKV_F16;
#define PKV_LATENT(RANK, ROPE) \
    if (p->rank == RANK && p->rope == ROPE) return launch_shape<RANK, ROPE>(a, f16, fp8, p->phases, stream);
    PKV_LATENT(512, 64) PKV_LATENT(256, 64) PKV_LATENT(128, 64) PKV_LATENT(128, 32) PKV_LATENT(64, 64) PKV_LATENT(64, 32)
    PKV_LATENT(1024, 64) PKV_LATENT(512, 128)
#undef PKV_LATENT
    return CRIT_PKV_E_GEOMETRY;
}

}   // namespace pkv
