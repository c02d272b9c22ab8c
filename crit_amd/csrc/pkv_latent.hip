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
    int tile_rows;      // the caller's choice: 0 (the geometry decides), 16, 128
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

// -- many heads: 128 query rows a workgroup -----------------------------------------------------------------------------
// With 128 heads a launch spends 2 (2 R + P) flops a query row and position on (R + P) e bytes: it is bound by the matrix
// pipe and by what LDS can feed it as much as by HBM. The kernel above reads a step's cache rows from LDS once for every
// 16 query rows, and every workgroup of a (row, partition) stages them again. This one holds 128 query rows in a
// workgroup of four wavefronts, one a SIMD with 512 registers each, on v_mfma_f32_32x32x16:
//   scores  S^T = K Q^T      wavefront w takes rows 32 w .. 32 w + 31: A = cache rows (a lane: position n32, 8 values
//                            of half h of the k-step), B = its queries, all (R + P) / 16 k-steps in 144 registers. Two
//                            chains of 18 products: a product every 32 clocks cannot wait for the one before it.
//   softmax                  the wavefront's own 32 rows; the probabilities (16-bit, [row][position]) and each row's
//                            factor on its accumulators go to LDS for the others.
//   values  O^T += V^T P^T   wavefront w takes values 128 w .. 128 w + 127 of ALL 128 rows (256 accumulators): A = V^T
//                            by two ds_read_b64_tr_b16 an operand (4 positions of one value each), read once for four
//                            products; B = the four row blocks' probabilities from LDS. Splitting the values rather
//                            than the rows quarters the transposing reads, the slowest the LDS serves.
// The cache rows reach LDS without passing through registers (global_load_lds_dwordx4: there are none to spare) into a
// ring of four tiles of 32 positions, three in flight while one is multiplied; a wavefront sends nine loads a tile,
// spread between the products, because each holds the wavefront until the memory pipe has taken it. Two barriers a
// step: the tile has landed; the probabilities are written.
//
// A tile in LDS: the latents as [32 positions][R values] (rows of 2 R bytes, no padding) and behind them the rotary keys
// as [32][P]. The DMA writes lane i's 16 bytes at byte 16 i of what an instruction fills, but a lane may fetch any 16
// bytes, so the 16-byte chunks of a row are stored permuted: chunk c of position n at place c ^ (4 (n & 3) + ((n >> 2)
// & 3)) of the latent row (c ^ ((n >> 1) & 7) of the rotary row). The score product's operand read (16 lanes: 16
// positions, one chunk each) and the transposing read of the values (a half-wave: 4 positions x 64 bytes) then both
// fall on all 64 banks once (the bank-conflict counter read zero while the tiles were all the LDS traffic; the 8-byte
// writes of the probabilities meet two to a bank).
//
// The softmax keeps a row's reference maximum until the running maximum exceeds it by more than kLazyHeads (base 2), so
// the 256 accumulators are rescaled on few steps; the decision is the row's own, from its own scores in step order.
// A row's bits depend on its query, its positions, `piece` and `partitions` only, as above (they differ from the
// kernel above: which of the two serves a launch follows from tile_rows, the heads, the shape and the page alone, never
// from the batch). The partials are stored as the registers hold them (whole kilobytes a store) and merged by a kernel
// of their own, below.
//
// Measured on MI355X, 64 rows of one token at contexts ~U[1024, 8192], 128 heads, BF16: 127-130 us (the kernel above:
// 259 us). With every phase after the other (142 us) a step of 32 positions took about 4,600 clocks against 2,176 of
// matrix instructions (scores 1,800, softmax and the probabilities' way through LDS 750, values 1,900, barriers 300),
// so 16-bit rows now send a step's value products out one step later, with the next step's softmax between them. A
// unit's start (ranking the rows, the table, the queries: 36 gathers of 32 rows x 32 bytes a wavefront) and end (256
// KB of partials) are another 38,000. With one workgroup a compute unit nothing hides either, so launches of a few rows
// are slower than with the small tiles (1 row: 67 us against 40): tile_rows = 16 asks for those. E4M3 rows (see the
// kernel's constants): 158 us.
constexpr float kLazyHeads = 8.0f;
constexpr int kHeadsRows = 128;      // query rows a workgroup of the many-heads kernel holds
constexpr int kRowsToAnXcd = 16;     // launches of that many batch rows or more keep a row's units on one XCD

template <bool F16>
PKV_DEV f32x16 mfma_32(u32x4 a, u32x4 b, f32x16 c) {
    if constexpr (F16) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
}
// (The loads are spelled in assembly so that the compiler neither counts them nor waits for them: the waits are the
// kernel's own, and those and the barrier are "memory" clobbers, which keeps a tile's LDS reads behind them.)
// 64 lanes x 16 bytes from base + offset (a lane's own) to LDS bytes lds .. lds + 1023.
PKV_DEV void dma_row(uint32_t offset, const uint8_t* base, unsigned lds) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(offset), "s"(base), "s"(lds));
}
PKV_DEV void dma_any(const uint8_t* from, unsigned lds) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(from), "s"(lds));
}
PKV_DEV void dma_word(const float* from, unsigned lds) {      // 4 bytes a lane, to LDS bytes lds + 4 lane
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(from), "s"(lds));
}
template <int N>
PKV_DEV void wait_loads() {
    static_assert(N >= 0 && N < 64, "vmcnt is six bits");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// The score products and their operand reads are spelled out too, with the accumulators in ordinary registers (the
// compiler would put them where the value accumulators are and move 16 of those out and back every step) and the waits
// counted by hand: `ahead` reads are in flight behind the one a product needs.
template <bool F16>
PKV_DEV void score_product(f32x16& c, const u32x4& a, const u32x4& b) {
    if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}
template <bool F16>
PKV_DEV void score_product_first(f32x16& c, const u32x4& a, const u32x4& b) {      // (a chain's first: onto zeros)
    if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
}
template <int OFFSET>
PKV_DEV void lds_read16(u32x4& to, uint32_t at) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(to) : "v"(at), "n"(OFFSET));
}
template <int AHEAD>
PKV_DEV void lds_arrived(u32x4& x) {      // (the operand is named so that its use cannot move above the wait)
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x) : "n"(AHEAD));
}

template <int R, int P, bool F16, bool FP8>
__global__ __launch_bounds__(256, 1) void latent_heads_kernel(LatentArgs a) {
    static_assert(R == 512 && P == 64, "rows of 1,024 + 128 bytes");
    constexpr int W = R + P, KS = W / 16, KSL = R / 16, NB = R / 32;      // k-steps of the scores (the first KSL the latent's); value blocks
    // E4M3 caches: the codes land in a ring of three raw tiles (a wavefront's eight rows side by side, as they lie in
    // HBM) and the wavefront that fetched them writes them out as 16-bit values, exactly, into one of two tiles of the
    // layout the products read, one step ahead of its use; a row's scales travel the same way.
    constexpr int MAIN = 32 * R * 2, TILE = MAIN + 32 * P * 2, NSTAGE = FP8 ? 2 : 4;
    constexpr int RAW = 32 * W, NRAW = 3, CPR = W / 16;      // a raw tile's bytes; raw tiles; 16-byte chunks of a row of codes
    // loads a wavefront issues a tile: its 8 latent rows and the rotary keys of the same rows (16-bit); 4.5 KB of codes
    // and the rows' scales (E4M3)
    constexpr int LPT = FP8 ? 6 : 9;
    __shared__ __align__(1024) uint8_t ring[NSTAGE * TILE];
    __shared__ __align__(1024) uint8_t raw[FP8 ? NRAW * RAW : 16];
    __shared__ float s_raw_scale[FP8 ? NRAW : 1][4][16];             // [raw tile][wavefront][latent, rotary][its row]
    __shared__ __align__(16) float s_scale[FP8 ? 2 : 1][2][32];      // [tile][latent, rotary][position]
    __shared__ __align__(16) uint8_t s_prob[kHeadsRows * 64];      // the step's probabilities, 16-bit [row][position]
    __shared__ float s_alpha[kHeadsRows];                           // the step's factor on each row's accumulators

    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, n32 = lane & 31, h = lane >> 5;
    // Workgroups go to the XCDs in turn (workgroup i to XCD i mod 8), and the tile groups of one (row, partition) pair
    // take consecutive places of one XCD, whose L2 then serves the pair's cache rows to all of them. Launches of 16 batch
    // rows or more deal whole rows to the XCDs (a row's partitions read the same queries, which one L2 then fetches
    // once: 142 against 165 us for 64 rows of 128 heads); smaller ones deal the pairs, or XCDs would idle.
    // Workgroups start in grid order and a compute unit holds one: a launch ends when the last one does, so the longest
    // rows go first (ranked here, lane i holding row i: launches of up to 64 rows; larger ones keep the caller's order).
    const int64_t place = blockIdx.x >> 3;
    const int group = (int)(place % a.tiles);
    int b, r;
    if (a.n_rows >= kRowsToAnXcd) {
        const int64_t pair = place / a.tiles;
        b = (int)(pair % a.gy), r = (int)(pair / a.gy) * 8 + (int)(blockIdx.x & 7);
        if (r >= a.n_rows) return;
    } else {
        const int64_t pair = (place / a.tiles) * 8 + (int64_t)(blockIdx.x & 7);
        if (pair >= a.pairs) return;
        b = (int)(pair % a.gy), r = (int)(pair / a.gy);
    }
    if (a.n_rows <= 64 && a.n_rows > 1) {
        // (keys are distinct: the length, then the lower index first)
        uint64_t mine = 0;
        if (lane < a.n_rows) {
            const int c = a.counts ? min(a.counts[lane], a.columns) : a.columns;
            const int64_t f = a.firsts[lane];
            mine = ((uint64_t)((f < 0 ? 0 : (f > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : f)) + c) << 8) + (uint64_t)(64 - lane);
        }
        const uint32_t lo = (uint32_t)mine, hi = (uint32_t)(mine >> 32);
        int rank = 0;
        for (int j = 0; j < a.n_rows; ++j) {
            const uint64_t other = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)hi, j) << 32) | (uint32_t)__builtin_amdgcn_readlane((int)lo, j);
            rank += other > mine ? 1 : 0;
        }
        r = __builtin_ctzll(__ballot(lane < a.n_rows && rank == r));
    }
    int count = a.columns;
    if (a.counts) count = min(a.counts[r], a.columns);
    const int H = a.heads;
    const int live_rows = count * H;
    if (group * kHeadsRows >= live_rows) return;
    const int64_t first64 = a.firsts[r];
    const int first = (int)(first64 < 0 ? 0 : (first64 > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : first64));
    const int c_hi = (min((group + 1) * kHeadsRows, live_rows) - 1) / H + 1;      // columns the group's rows reach
    const int n_keys = min(first + c_hi, a.max_keys);
    const int n_pieces = (n_keys + a.piece - 1) / a.piece;
    if (b >= n_pieces) return;
    const int64_t trow = (int64_t)a.rows[(int64_t)r * a.rows_step] * a.tab_stride;
    const int start = a.starts[r];

    // The unit's tiles: tile t is step t % spp of piece b + (t / spp) parts.
    const int spp = a.piece / 32;
    int n_tiles;
    {
        const int whole = (n_pieces - 1 - b) / a.parts;      // the unit's pieces before its last
        const int last_piece = b + whole * a.parts;
        const int left = n_keys - last_piece * a.piece;      // positions of the last piece (>= 1)
        n_tiles = whole * spp + min(spp, (left + 31) / 32);
    }

    // -- staging. Wavefront w fills rows 8 w .. 8 w + 7 of a tile: one load a latent row (lane i: the chunk that belongs
    // at place i), one for the rotary keys of the eight rows (lane i: row i / 8, the chunk that belongs at place i % 8).
    // A wavefront's eight rows are neighbours in one page (pages are multiples of 16 positions), so it needs one page
    // table entry a tile: the lanes hold, for 64 tiles at a time, each tile's first position and the slot that
    // position 0 would have in the page of the wavefront's rows, and a step takes its own by v_readlane: no load inside
    // the loop waits on the table.
    const unsigned ring_at = (unsigned)(uintptr_t)ring;
    const int half_row = 16 * (wave >> 1);
    // (What a lane derives from its number is derived again in every step, from a copy of the number the compiler cannot
    // see through: kept across the loop, the few dozen addresses below would push the queries out of the registers.)
    int ln = lane;
    int tile_pos = 0, tile_slot = 0, held_from = 0;
    auto hold_tiles = [&](int from) __attribute__((always_inline)) {
        const int tt = min(from + lane, n_tiles - 1);
        const int pc = tt / spp;
        const int base = (b + pc * a.parts) * a.piece + (tt - pc * spp) * 32;
        const int p0 = min(base + half_row, n_keys - 1);
        const int page_index = (int)div32(a.page_div, (uint32_t)p0);
        const int entry = a.tables[trow + (page_index < a.tab_width ? page_index : a.tab_width - 1)];
        tile_pos = base, tile_slot = (entry - page_index) * a.page, held_from = from;
    };
    hold_tiles(0);
    // plan: where tile t comes from and goes to (past the unit's last tile: that one again, so that every wait counts the
    // same loads); returns its first position. send: load k of the planned tile's nine. Inside the loop the loads go out
    // between the score products, a few products apart: issued back to back they would hold the wavefront, and its SIMD's
    // matrix pipe with it, until the memory pipe has taken them all.
    const uint8_t* plan_row0 = a.cache;
    const float* plan_scale0 = a.scales;
    int plan_room = 0;
    unsigned plan_to = 0, plan_scale_to = 0;
    const unsigned raw_at = (unsigned)(uintptr_t)raw, raw_scale_at = (unsigned)(uintptr_t)&s_raw_scale[0][0][0];
    auto plan = [&](int t, int stage) __attribute__((always_inline)) -> int {
        t = t < n_tiles ? t : n_tiles - 1;
        if (t - held_from >= 64) hold_tiles(held_from + 64);
        const int base = __builtin_amdgcn_readlane(tile_pos, t - held_from);
        const int page_slot = __builtin_amdgcn_readlane(tile_slot, t - held_from);
        const int n0 = min(base + 8 * wave, n_keys - 1);
        plan_room = n_keys - 1 - n0;      // rows after the wavefront's first that are their own (the others repeat the last position)
        if constexpr (FP8) {
            plan_row0 = a.cache + (int64_t)(page_slot + n0) * W;
            plan_scale0 = a.scales + (int64_t)(page_slot + n0) * a.scales_per_row;
            plan_to = raw_at + (unsigned)(stage * RAW + wave * (8 * W));
            plan_scale_to = raw_scale_at + (unsigned)((stage * 4 + wave) * 64);
        } else {
            plan_row0 = a.cache + (int64_t)(page_slot + n0) * (W * 2);
            plan_to = ring_at + (unsigned)(stage * TILE);
        }
        return base;
    };
    auto send = [&](auto kc) __attribute__((always_inline)) {
        constexpr int k = decltype(kc)::value;
        if constexpr (FP8) {
            // (chunk c of the wavefront's 288: row c / 36 of its eight; the last load fills half a kilobyte)
            if constexpr (k < 5) {
                const int c = 64 * k + ln;
                if (k < 4 || ln < 32) {
                    const int row = c / CPR;
                    dma_any(plan_row0 + (uint32_t)(min(row, plan_room) * W + (c - row * CPR) * 16), plan_to + (unsigned)(k * 1024));
                }
            } else if constexpr (k == 5) {
                if (ln < 16) dma_word(plan_scale0 + min(ln & 7, plan_room) * a.scales_per_row + (ln >> 3) * (a.scales_per_row - 1), plan_scale_to);
            }
        } else if constexpr (k < 8) {
            const uint32_t place = (uint32_t)(ln ^ ((2 * wave + k / 4) & 3)) * 16u;
            dma_row(place ^ (uint32_t)(64 * (k & 3)), plan_row0 + min(k, plan_room) * (W * 2), plan_to + (unsigned)((8 * wave + k) * (R * 2)));
        } else {
            const int tail_row = ln >> 3;
            const uint32_t tail_at = (uint32_t)(R * 2 + 16 * ((ln & 7) ^ (((8 * wave + tail_row) >> 1) & 7)));
            dma_any(plan_row0 + (uint32_t)(min(tail_row, plan_room) * (W * 2)) + tail_at, plan_to + (unsigned)(MAIN + wave * 1024));
        }
    };
    auto issue = [&](int t, int stage) __attribute__((always_inline)) -> int {
        const int base = plan(t, stage);
        static_for<LPT>(send);
        return base;
    };

    // The lane's query row: column n32 of its wavefront's score tile.
    const int j0 = group * kHeadsRows + wave * 32;
    const int jq = j0 + n32, colq = jq / H, headq = jq - colq * H;
    const bool liveq = colq < count;
    const int lim = liveq ? first + colq : -1;
    const int unmasked = min(first + j0 / H + 1, n_keys);      // positions below it are seen by every live row of the wavefront

    int base = issue(0, 0);
    u32x4 bq[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        bq[ks] = u32x4{0u, 0u, 0u, 0u};
        if (liveq) bq[ks] = *reinterpret_cast<const u32x4*>(a.q + ((int64_t)(start + colq) * a.q_st + (int64_t)headq * a.q_sh) * 2 + ks * 32 + h * 16);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" ::"v"(bq[ks].x), "v"(bq[ks].y), "v"(bq[ks].z), "v"(bq[ks].w));
    // (the queries are waited for here, with the first tile; the next two tiles go out behind them)
    int base1 = issue(1, 1), base2 = FP8 ? issue(2, 2) : 0;
    // E4M3: the wavefront's rows of raw tile `from`, as 16-bit values in tile `to` (a lane: 16 codes a turn).
    // (In five parts, without a branch, so that a part can go between the value products: the last part's upper lanes
    // repeat the lower ones' chunks, and every quarter-wave copies the scales.)
    auto convert_part = [&](auto jc, int from, int to) __attribute__((always_inline)) {
        if constexpr (FP8) {
            constexpr int j = decltype(jc)::value;
            asm volatile("" : "+v"(ln));
            const uint8_t* codes_at = raw + from * RAW + wave * (8 * W);
            uint8_t* tile_to = ring + to * TILE;
            {
                const int c = 64 * j + (j < 4 ? ln : (ln & 31));
                {
                    const int row = c / CPR, cj = c - row * CPR, n = 8 * wave + row;
                    const u32x4 codes = *reinterpret_cast<const u32x4*>(codes_at + c * 16);
                    const uint32_t w[4] = {codes.x, codes.y, codes.z, codes.w};
                    uint32_t o[8];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        if constexpr (F16) {
                            const f32x2 lo = e4m3_pair<false>(w[k]), hi = e4m3_pair<true>(w[k]);
                            o[2 * k] = pair16<true>(lo.x, lo.y), o[2 * k + 1] = pair16<true>(hi.x, hi.y);
                        } else {
                            const u32x2 both = codes4_to_pairs<1>(w[k]);
                            o[2 * k] = both.x, o[2 * k + 1] = both.y;
                        }
                    }
                    // (16-bit chunks 2 cj and 2 cj + 1 of position n, each at its permuted place)
                    const bool latent = cj < KSL;
                    const uint32_t turn = latent ? (uint32_t)(4 * (n & 3) + ((n >> 2) & 3)) : (uint32_t)((n >> 1) & 7);
                    uint8_t* row_at = tile_to + (latent ? n * (R * 2) : MAIN + n * (P * 2));
                    const uint32_t chunk = (uint32_t)(latent ? 2 * cj : 2 * (cj - KSL));
                    *reinterpret_cast<u32x4*>(row_at + 16 * (chunk ^ turn)) = u32x4{o[0], o[1], o[2], o[3]};
                    *reinterpret_cast<u32x4*>(row_at + 16 * ((chunk + 1) ^ turn)) = u32x4{o[4], o[5], o[6], o[7]};
                }
            }
            if constexpr (j == 4) s_scale[to][(ln >> 3) & 1][8 * wave + (ln & 7)] = s_raw_scale[from][wave][ln & 15];
        }
    };
    auto convert = [&](int from, int to) __attribute__((always_inline)) {
        static_for<5>([&](auto jc) __attribute__((always_inline)) { convert_part(jc, from, to); });
    };
    if constexpr (FP8) {
        wait_loads<2 * LPT>();      // (its own rows of the first tile are all a wavefront converts: no barrier)
        convert(0, 0);
    }
    int raw_stage = 0;      // E4M3: the raw tile that held tile t (tile t + 3 goes there)

    float m = -INFINITY, l = 0.0f;
    f32x16 acc[4][4];      // [block of 32 values][block of 32 query rows]
#pragma unroll
    for (int vb = 0; vb < 4; ++vb)
#pragma unroll
        for (int hb = 0; hb < 4; ++hb)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[vb][hb][v] = 0.0f;

    if constexpr (FP8) {
        for (int t = 0; t < n_tiles; ++t) {
            const int stage = t & (NSTAGE - 1);
            // 16-bit: the tile's loads of this wavefront have landed, those of the next two may be in flight. E4M3: the next
            // tile's have (it is converted at the end of this step), the one after may be in flight.
            wait_loads<FP8 ? LPT : 2 * LPT>();
            lds_barrier();              // everybody's have, and nobody reads the tile before any more, nor the last probabilities
            const int base3 = plan(t + 3, FP8 ? raw_stage : (t + 3) & (NSTAGE - 1));
            const uint8_t* tile = ring + stage * TILE;
            // Operand addresses inside a tile (see the layout above), from the opaque copy of the number of the lane.
            asm volatile("" : "+v"(ln));
            const int n32 = ln & 31, h = ln >> 5;
            const int fk = 4 * (n32 & 3) + ((n32 >> 2) & 3);
            const uint32_t k_lane = (uint32_t)(n32 * (R * 2) + 16 * ((fk ^ h) & 15));                       // ^ 32 i for k-step i of the latent
            const uint32_t t_lane = (uint32_t)(MAIN + n32 * (P * 2) + 16 * ((h ^ (n32 >> 1)) & 7));         // ^ 32 i for k-step i of the rotary key
            // The values: the wavefront's 128 of them. For block vb of 32 values and k-step g of 16 positions the lane's operand
            // is positions 16 g + 8 h + 4 e + (0 .. 3), e = 0, 1: two transposing reads, lane 4 j + c of a 16-lane group pointing
            // at position j's values 4 c .. 4 c + 3.
            const int i16 = ln & 15, mh = (ln >> 4) & 1;
            const uint32_t v_lane = (uint32_t)((8 * h + (i16 >> 2)) * (R * 2) + 256 * wave + 8 * (i16 & 1));
            const uint32_t v_low = (uint32_t)(2 * mh + ((i16 & 3) >> 1));      // the chunk's low two bits, ^ ((2 h + e) & 3)
            uint8_t* p_mine = s_prob + (wave * 32 + n32) * 64 + 8 * h;           // + 16 (q ^ p_turn): positions 8 q + 4 h .. + 3
            const uint32_t p_turn = (uint32_t)((n32 >> 2) & 3);
            const uint8_t* p_read = s_prob + n32 * 64;                           // + 2048 hb + 16 ((2 g + h) ^ p_turn)

            // -- scores of the wavefront's 32 rows: 36 products in two chains (even and odd ones: a product every 32 clocks
            // cannot wait for the one before it), the operand of each read RING - 1 products ahead, five of the tile's loads
            // sent out in between
            // (E4M3: the rotary keys' products, which take a scale of their own, in a chain of their own, every ninth)
            f32x16 s, s2, s3;
            {
                constexpr int RING = 6;
                u32x4 ka[RING];
                const uint32_t tile_at = (uint32_t)(uintptr_t)tile;
                // the latent's k-steps in the order 0, 8, 16, 24, 1, 9, ...: four share an address register
                uint32_t k_at = 0;
                auto read_k = [&](auto ic) __attribute__((always_inline)) {
                    constexpr int i = decltype(ic)::value;
                    constexpr bool rotary = FP8 ? i % 9 == 8 : i >= KSL;
                    constexpr int at = FP8 ? (rotary ? i / 9 : i - i / 9) : (rotary ? i - KSL : i);
                    if constexpr (!rotary) {
                        constexpr int lo = at / 4, hi = at % 4;      // k-step lo + 8 hi
                        if constexpr (hi == 0) k_at = tile_at + (k_lane ^ (uint32_t)(32 * lo));
                        lds_read16<256 * hi>(ka[i % RING], k_at);
                    } else {
                        lds_read16<0>(ka[i % RING], tile_at + (t_lane ^ (uint32_t)(32 * at)));
                    }
                };
                static_for<RING - 1>([&](auto ic) __attribute__((always_inline)) { read_k(ic); });
                static_for<KS>([&](auto ic) __attribute__((always_inline)) {
                    constexpr int i = decltype(ic)::value;
                    if constexpr (i + RING - 1 < KS) read_k(std::integral_constant<int, i + RING - 1>{});
                    if constexpr (i % 8 == 2) send(std::integral_constant<int, i / 8>{});
                    constexpr int ahead = KS - 1 - i < RING - 1 ? KS - 1 - i : RING - 1;
                    lds_arrived<ahead>(ka[i % RING]);
                    constexpr bool rotary = FP8 ? i % 9 == 8 : i >= KSL;
                    constexpr int at = FP8 ? (rotary ? i / 9 : i - i / 9) : (rotary ? i - KSL : i);
                    constexpr int ks = rotary ? KSL + at : at / 4 + 8 * (at % 4);
                    // (a chain's first product onto zeros)
                    if constexpr (FP8 && rotary && at == 0) score_product_first<F16>(s3, ka[i % RING], bq[ks]);
                    else if constexpr (FP8 && rotary) score_product<F16>(s3, ka[i % RING], bq[ks]);
                    else if constexpr (i == 0) score_product_first<F16>(s, ka[i % RING], bq[ks]);
                    else if constexpr (i == 1) score_product_first<F16>(s2, ka[i % RING], bq[ks]);
                    else if constexpr ((FP8 ? at : i) % 2 == 0) score_product<F16>(s, ka[i % RING], bq[ks]);
                    else score_product<F16>(s2, ka[i % RING], bq[ks]);
                });
                // (the products' results are read by vector instructions next)
                if constexpr (FP8) asm volatile("s_nop 15\n\ts_nop 15" : "+v"(s), "+v"(s2), "+v"(s3));
                else asm volatile("s_nop 15\n\ts_nop 15" : "+v"(s), "+v"(s2));
            }
            // -- softmax of the lane's row over its 16 positions of the tile (the other half-wave holds the other 16): the
            // lane holds positions 8 (v / 4) + 4 h + v % 4
            const bool masked = base + 32 > unmasked;      // (the same for the whole wavefront)
            float x[16];
            if constexpr (FP8) {      // (the scales of the lane's positions: the latent's, the rotary key's)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f32x4 scale0 = *reinterpret_cast<const f32x4*>(&s_scale[stage][0][8 * q + 4 * h]);
                    const f32x4 scale1 = *reinterpret_cast<const f32x4*>(&s_scale[stage][1][8 * q + 4 * h]);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        x[4 * q + e] = __builtin_fmaf(s[4 * q + e] + s2[4 * q + e], scale0[e], s3[4 * q + e] * scale1[e]) * a.sscale;
                }
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v) x[v] = (s[v] + s2[v]) * a.sscale;
            }
            if (masked) {
                const int seen = min(lim, n_keys - 1) - base - 4 * h;      // position 8 (v / 4) + v % 4 of the lane's is seen up to this
#pragma unroll
                for (int v = 0; v < 16; ++v) x[v] = 8 * (v / 4) + v % 4 <= seen ? x[v] : -INFINITY;
            }
            float top = x[0];
#pragma unroll
            for (int v = 1; v < 16; ++v) top = __builtin_fmaxf(top, x[v]);
            {
                const int w = (int)f2u(top);
                const auto both = __builtin_amdgcn_permlane32_swap(w, w, false, false);
                top = __builtin_fmaxf(u2f((uint32_t)both[0]), u2f((uint32_t)both[1]));
            }
            const float m_new = top > m + kLazyHeads ? top : m;      // (a NaN score: the comparison fails, the NaN reaches the sum)
            const float sub = m_new == -INFINITY ? 0.0f : m_new;
            const float alpha = exp2_fast(m - sub);
            m = m_new;
            float p[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) p[v] = exp2_fast(x[v] - sub);
            const float sum = (((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]))) +
                              (((p[8] + p[9]) + (p[10] + p[11])) + ((p[12] + p[13]) + (p[14] + p[15])));
            l = __builtin_fmaf(l, alpha, sum);
            if constexpr (FP8) {      // a value is its code times its position's latent scale: the scale rides on the probability
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f32x4 scale0 = *reinterpret_cast<const f32x4*>(&s_scale[stage][0][8 * q + 4 * h]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) p[4 * q + e] *= scale0[e];
                }
            }
            // The probabilities and the row's factor go to the other wavefronts through LDS: each multiplies the values it
            // owns by the probabilities of all 128 rows.
#pragma unroll
            for (int q = 0; q < 4; ++q)
                *reinterpret_cast<u32x2*>(p_mine + 16 * ((uint32_t)q ^ p_turn)) =
                    u32x2{pair16<F16>(p[4 * q], p[4 * q + 1]), pair16<F16>(p[4 * q + 2], p[4 * q + 3])};
            if (h == 0) s_alpha[wave * 32 + n32] = alpha;
            lds_barrier();
            float factor[4];
#pragma unroll
            for (int hb = 0; hb < 4; ++hb) factor[hb] = s_alpha[hb * 32 + n32];
            if (__ballot(factor[0] != 1.0f || factor[1] != 1.0f || factor[2] != 1.0f || factor[3] != 1.0f) != 0ull) {
                // (x 1 is exact: the accumulators move only when some row's reference did; spelled out so that they stay
                // where the matrix pipe keeps them, and the last product that wrote them is a whole score phase back)
                static_for<16>([&](auto bc) __attribute__((always_inline)) {
                    constexpr int vb = decltype(bc)::value / 4, hb = decltype(bc)::value % 4;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        float e = acc[vb][hb][v], tmp;
                        asm volatile("v_accvgpr_read_b32 %0, %1\n\tv_mul_f32 %0, %0, %2\n\tv_accvgpr_write_b32 %1, %0" : "=&v"(tmp), "+a"(e) : "v"(factor[hb]));
                        acc[vb][hb][v] = e;
                    }
                });
            }
            // -- values: operand i = (k-step g = i / 4, block vb = i % 4) of V^T against the four row blocks' probabilities
            const int next_raw = raw_stage == NRAW - 1 ? 0 : raw_stage + 1;
            {
                constexpr int RING = 4, NOPS = 8;
                u32x4 pb[4];      // the four row blocks' probabilities of the k-step being multiplied
                u32x2 va[RING][2];
                auto read_p = [&](auto gc) __attribute__((always_inline)) {
                    constexpr int g = decltype(gc)::value;
#pragma unroll
                    for (int hb = 0; hb < 4; ++hb)
                        pb[hb] = *reinterpret_cast<const u32x4*>(p_read + 2048 * hb + 16 * ((uint32_t)(2 * g + h) ^ p_turn));
                };
                read_p(std::integral_constant<int, 0>{});
                auto read_v = [&](auto ic) __attribute__((always_inline)) {
                    constexpr int i = decltype(ic)::value;
                    constexpr int g = i / 4, vb = i % 4;
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        const uint32_t at = v_lane + 64u * (uint32_t)(vb ^ (i16 >> 2)) + 16u * (v_low ^ (uint32_t)((2 * h + e) & 3));
                        va[i % RING][e] = lds_transposed(tile + at + (16 * g + 4 * e) * (R * 2));
                    }
                };
                static_for<RING - 1>([&](auto ic) __attribute__((always_inline)) { read_v(ic); });
                __builtin_amdgcn_sched_group_barrier(0x100, 4 + 2 * (RING - 1), 0);
                __builtin_amdgcn_sched_barrier(0);
                static_for<NOPS / 2>([&](auto sc) __attribute__((always_inline)) {
                    constexpr int sec = decltype(sc)::value;
                    if constexpr (!FP8 || sec == 0) send(std::integral_constant<int, 5 + sec>{});
                    if constexpr (sec == 2) {      // (the first k-step's products have been issued: their operands were read at issue)
                        read_p(std::integral_constant<int, 1>{});
                        __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    static_for<2>([&](auto jc) __attribute__((always_inline)) {
                        constexpr int i = 2 * sec + decltype(jc)::value;
                        constexpr int g = i / 4, vb = i % 4;
                        if constexpr (i + RING - 1 < NOPS) read_v(std::integral_constant<int, i + RING - 1>{});
                        const u32x4 av = {va[i % RING][0].x, va[i % RING][0].y, va[i % RING][1].x, va[i % RING][1].y};
#pragma unroll
                        for (int hb = 0; hb < 4; ++hb) acc[vb][hb] = mfma_32<F16>(av, pb[hb], acc[vb][hb]);
                    });
                    // (the next tile's codes become values between the products: a part a section, two in the last)
                    convert_part(sc, next_raw, stage ^ 1);
                    if constexpr (sec == 3) convert_part(std::integral_constant<int, 4>{}, next_raw, stage ^ 1);
                    static_for<2>([&](auto jc) __attribute__((always_inline)) {
                        constexpr int i = 2 * sec + decltype(jc)::value;
                        if constexpr (i + RING - 1 < NOPS) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                    });
                    __builtin_amdgcn_sched_barrier(0);
                });
            }
            raw_stage = next_raw;
            base = base1, base1 = base2, base2 = base3;
        }
    } else {
        // 16-bit rows: the same operations on the same numbers in a pipeline of one step: a step's value products go out
        // one step later, together with the next step's softmax, whose vector work then runs in their shadow instead of
        // with the matrix pipe idle. A tile therefore stays in the ring one step longer, and two tiles are in flight
        // instead of three. Barriers: A, the tile has landed and the last probabilities are written; B, everybody has read
        // those probabilities, the next may be written.
        struct Lane {
            int h, i16;
            uint32_t k_lane, t_lane, v_lane, v_low, p_turn;
            uint8_t* p_mine;
            const uint8_t* p_read;
        };
        auto lane_of = [&]() __attribute__((always_inline)) -> Lane {
            Lane L;
            const int n32 = ln & 31, h = ln >> 5;
            const int fk = 4 * (n32 & 3) + ((n32 >> 2) & 3);
            L.h = h, L.i16 = ln & 15;
            L.k_lane = (uint32_t)(n32 * (R * 2) + 16 * ((fk ^ h) & 15));
            L.t_lane = (uint32_t)(MAIN + n32 * (P * 2) + 16 * ((h ^ (n32 >> 1)) & 7));
            const int mh = (ln >> 4) & 1;
            L.v_lane = (uint32_t)((8 * h + (L.i16 >> 2)) * (R * 2) + 256 * wave + 8 * (L.i16 & 1));
            L.v_low = (uint32_t)(2 * mh + ((L.i16 & 3) >> 1));
            L.p_mine = s_prob + (wave * 32 + n32) * 64 + 8 * h;
            L.p_turn = (uint32_t)((n32 >> 2) & 3);
            L.p_read = s_prob + n32 * 64;
            return L;
        };
        // (Five of them are kept; the rest, and what a step derives from any, is derived again in every step from copies
        // the compiler cannot see through, or it would keep all of that too and push the queries out of the registers.)
        const Lane lane_kept = lane_of();
        auto lane_now = [&]() __attribute__((always_inline)) -> Lane {
            asm volatile("" : "+v"(ln));
            Lane L = lane_of();
            L.k_lane = lane_kept.k_lane, L.t_lane = lane_kept.t_lane, L.v_lane = lane_kept.v_lane, L.v_low = lane_kept.v_low,
            L.p_turn = lane_kept.p_turn;
            asm volatile("" : "+v"(L.k_lane), "+v"(L.t_lane), "+v"(L.v_lane), "+v"(L.v_low), "+v"(L.p_turn));
            return L;
        };
        f32x16 s, s2;
        auto scores = [&](const uint8_t* tile, const Lane& L) __attribute__((always_inline)) {
            constexpr int RING = 6;
            u32x4 ka[RING];
            const uint32_t tile_at = (uint32_t)(uintptr_t)tile;
            uint32_t k_at = 0;
            auto read_k = [&](auto ic) __attribute__((always_inline)) {
                constexpr int i = decltype(ic)::value;
                if constexpr (i < KSL) {
                    constexpr int lo = i / 4, hi = i % 4;      // k-step lo + 8 hi
                    if constexpr (hi == 0) k_at = tile_at + (L.k_lane ^ (uint32_t)(32 * lo));
                    lds_read16<256 * hi>(ka[i % RING], k_at);
                } else {
                    lds_read16<0>(ka[i % RING], tile_at + (L.t_lane ^ (uint32_t)(32 * (i - KSL))));
                }
            };
            static_for<RING - 1>([&](auto ic) __attribute__((always_inline)) { read_k(ic); });
            static_for<KS>([&](auto ic) __attribute__((always_inline)) {
                constexpr int i = decltype(ic)::value;
                if constexpr (i + RING - 1 < KS) read_k(std::integral_constant<int, i + RING - 1>{});
                if constexpr (i % 8 == 2) send(std::integral_constant<int, i / 8>{});
                constexpr int ahead = KS - 1 - i < RING - 1 ? KS - 1 - i : RING - 1;
                lds_arrived<ahead>(ka[i % RING]);
                constexpr int ks = i < KSL ? i / 4 + 8 * (i % 4) : i;
                if constexpr (i == 0) score_product_first<F16>(s, ka[i % RING], bq[ks]);
                else if constexpr (i == 1) score_product_first<F16>(s2, ka[i % RING], bq[ks]);
                else if constexpr (i % 2 == 0) score_product<F16>(s, ka[i % RING], bq[ks]);
                else score_product<F16>(s2, ka[i % RING], bq[ks]);
            });
            asm volatile("s_nop 15\n\ts_nop 15" : "+v"(s), "+v"(s2));
        };
        // The softmax of a step in four parts (each goes behind a quarter of the value products), on x in place.
        float x[16], alpha = 1.0f, sub = 0.0f;
        auto soften = [&](auto part_c, auto mask_c, int base, const Lane& L) __attribute__((always_inline)) {
            constexpr int part = decltype(part_c)::value;
            if constexpr (part == 0) {
                if constexpr (decltype(mask_c)::value) {
                    const int seen = min(lim, n_keys - 1) - base - 4 * L.h;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const float y = (s[v] + s2[v]) * a.sscale;
                        x[v] = 8 * (v / 4) + v % 4 <= seen ? y : -INFINITY;
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v) x[v] = (s[v] + s2[v]) * a.sscale;
                }
            } else if constexpr (part == 1) {
                float top = x[0];
#pragma unroll
                for (int v = 1; v < 16; ++v) top = __builtin_fmaxf(top, x[v]);
                const int w = (int)f2u(top);
                const auto both = __builtin_amdgcn_permlane32_swap(w, w, false, false);
                top = __builtin_fmaxf(u2f((uint32_t)both[0]), u2f((uint32_t)both[1]));
                const float m_new = top > m + kLazyHeads ? top : m;
                sub = m_new == -INFINITY ? 0.0f : m_new;
                alpha = exp2_fast(m - sub);
                m = m_new;
            } else if constexpr (part == 2) {
#pragma unroll
                for (int v = 0; v < 16; ++v) x[v] = exp2_fast(x[v] - sub);
            } else {
                const float sum = (((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]))) +
                                  (((x[8] + x[9]) + (x[10] + x[11])) + ((x[12] + x[13]) + (x[14] + x[15])));
                l = __builtin_fmaf(l, alpha, sum);
            }
        };
        auto publish = [&](const Lane& L) __attribute__((always_inline)) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
                *reinterpret_cast<u32x2*>(L.p_mine + 16 * ((uint32_t)q ^ L.p_turn)) =
                    u32x2{pair16<F16>(x[4 * q], x[4 * q + 1]), pair16<F16>(x[4 * q + 2], x[4 * q + 3])};
            if (L.h == 0) s_alpha[wave * 32 + (ln & 31)] = alpha;
        };
        auto rescale = [&]() __attribute__((always_inline)) {
            float factor[4];
#pragma unroll
            for (int hb = 0; hb < 4; ++hb) factor[hb] = s_alpha[hb * 32 + (ln & 31)];
            if (__ballot(factor[0] != 1.0f || factor[1] != 1.0f || factor[2] != 1.0f || factor[3] != 1.0f) != 0ull) {
                static_for<16>([&](auto bc) __attribute__((always_inline)) {
                    constexpr int vb = decltype(bc)::value / 4, hb = decltype(bc)::value % 4;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        float e = acc[vb][hb][v], tmp;
                        asm volatile("v_accvgpr_read_b32 %0, %1\n\tv_mul_f32 %0, %0, %2\n\tv_accvgpr_write_b32 %1, %0" : "=&v"(tmp), "+a"(e) : "v"(factor[hb]));
                        acc[vb][hb][v] = e;
                    }
                });
            }
        };
        // The value products of the tile at `tile` (its probabilities are in LDS), four of the planned tile's loads sent
        // between them (SEND) and the softmax of the step at `base` in their shadow (SOFT).
        auto values = [&](const uint8_t* tile, const Lane& L, auto send_c, auto soft_c, auto mask_c, int base) __attribute__((always_inline)) {
            constexpr bool SEND = decltype(send_c)::value, SOFT = decltype(soft_c)::value;
            constexpr int RING = 4, NOPS = 8;
            u32x4 pb[4];
            u32x2 va[RING][2];
            auto read_p = [&](auto gc) __attribute__((always_inline)) {
                constexpr int g = decltype(gc)::value;
#pragma unroll
                for (int hb = 0; hb < 4; ++hb)
                    pb[hb] = *reinterpret_cast<const u32x4*>(L.p_read + 2048 * hb + 16 * ((uint32_t)(2 * g + L.h) ^ L.p_turn));
            };
            read_p(std::integral_constant<int, 0>{});
            auto read_v = [&](auto ic) __attribute__((always_inline)) {
                constexpr int i = decltype(ic)::value;
                constexpr int g = i / 4, vb = i % 4;
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const uint32_t at = L.v_lane + 64u * (uint32_t)(vb ^ (L.i16 >> 2)) + 16u * (L.v_low ^ (uint32_t)((2 * L.h + e) & 3));
                    va[i % RING][e] = lds_transposed(tile + at + (16 * g + 4 * e) * (R * 2));
                }
            };
            static_for<RING - 1>([&](auto ic) __attribute__((always_inline)) { read_v(ic); });
            __builtin_amdgcn_sched_group_barrier(0x100, 4 + 2 * (RING - 1), 0);
            __builtin_amdgcn_sched_barrier(0);
            static_for<NOPS / 2>([&](auto sc) __attribute__((always_inline)) {
                constexpr int sec = decltype(sc)::value;
                if constexpr (SEND) send(std::integral_constant<int, 5 + sec>{});
                if constexpr (sec == 2) {
                    read_p(std::integral_constant<int, 1>{});
                    __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
                static_for<2>([&](auto jc) __attribute__((always_inline)) {
                    constexpr int i = 2 * sec + decltype(jc)::value;
                    constexpr int vb = i % 4;
                    if constexpr (i + RING - 1 < NOPS) read_v(std::integral_constant<int, i + RING - 1>{});
                    const u32x4 av = {va[i % RING][0].x, va[i % RING][0].y, va[i % RING][1].x, va[i % RING][1].y};
#pragma unroll
                    for (int hb = 0; hb < 4; ++hb) acc[vb][hb] = mfma_32<F16>(av, pb[hb], acc[vb][hb]);
                });
                if constexpr (SOFT) soften(sc, mask_c, base, L);
                static_for<2>([&](auto jc) __attribute__((always_inline)) {
                    constexpr int i = 2 * sec + decltype(jc)::value;
                    if constexpr (i + RING - 1 < NOPS) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                    static_for<4>([&](auto) __attribute__((always_inline)) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        if constexpr (SOFT) {
                            __builtin_amdgcn_sched_group_barrier(0x002, sec == 0 && decltype(mask_c)::value ? 8 : 4, 0);
                            if constexpr (sec == 1 || sec == 2) __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);
                        }
                    });
                });
                __builtin_amdgcn_sched_barrier(0);
            });
        };
        const std::true_type yes;
        const std::false_type no;
        // step 0: no values yet
        {
            wait_loads<LPT>();
            lds_barrier();
            const int base2 = plan(2, 2);
            const Lane L = lane_now();
            scores(ring, L);
            static_for<4>([&](auto sc) __attribute__((always_inline)) {
                send(std::integral_constant<int, 5 + decltype(sc)::value>{});
                soften(sc, yes, base, L);
            });
            publish(L);
            base = base1, base1 = base2;
        }
        // A unit's steps come in the order of their positions: first those every row of the wavefront sees whole, then
        // the masked ones, each kind in a loop of its own (a branch around the products inside one loop sends the
        // accumulators to scratch).
        auto step = [&](int t, auto mask_c) __attribute__((always_inline)) {
            wait_loads<LPT>();      // the tile's loads of this wavefront have landed: those of the next may be in flight
            lds_barrier();          // A
            const int base2 = plan(t + 2, (t + 2) & (NSTAGE - 1));
            const Lane L = lane_now();
            scores(ring + (t & (NSTAGE - 1)) * TILE, L);
            rescale();
            values(ring + ((t - 1) & (NSTAGE - 1)) * TILE, L, yes, yes, mask_c, base);
            lds_barrier();          // B
            publish(L);
            base = base1, base1 = base2;
        };
        int t = 1;
        for (; t < n_tiles && base + 32 <= unmasked; ++t) step(t, no);
        for (; t < n_tiles; ++t) step(t, yes);
        lds_barrier();
        {
            const Lane L = lane_now();
            rescale();
            values(ring + ((n_tiles - 1) & (NSTAGE - 1)) * TILE, L, no, no, no, 0);
        }
    }
    wait_loads<0>();      // (the loads past the last tile: LDS must not be written for a workgroup that has gone)
    {
        const int w = (int)f2u(l);
        const auto both = __builtin_amdgcn_permlane32_swap(w, w, false, false);
        l = u2f((uint32_t)both[0]) + u2f((uint32_t)both[1]);
    }
    // The partial output as the registers hold it, a lane's four values side by side and the lanes in order (whole
    // kilobytes a store): [unit][partition][wavefront][value block][row block][v / 4][lane][4]; the merge below reads the
    // same way. (Rows past a window's last are stored too, and never read.)
    if (h == 0 && liveq) {
        const int64_t index = ((int64_t)((int64_t)r * a.columns + colq) * H + headq) * a.parts + b;
        a.pm[index] = m, a.pl[index] = l;
    }
    float* slab = a.po + ((((int64_t)r * a.tiles + group) * a.parts + b) * 4 + wave) * (int64_t)(kHeadsRows * R / 4) + lane * 4;
#pragma unroll
    for (int vb = 0; vb < 4; ++vb)
#pragma unroll
        for (int hb = 0; hb < 4; ++hb)
#pragma unroll
            for (int v4 = 0; v4 < 4; ++v4)
                *reinterpret_cast<float4*>(slab + ((vb * 4 + hb) * 4 + v4) * 256) =
                    make_float4(acc[vb][hb][4 * v4], acc[vb][hb][4 * v4 + 1], acc[vb][hb][4 * v4 + 2], acc[vb][hb][4 * v4 + 3]);
}

// The many-heads kernel's partitions merged: a workgroup of 64 threads folds, in partition order, one (value block, row
// block) pair of one wavefront's share of a unit, reading the partials as that wavefront stored them; the sink last.
template <int R>
__global__ __launch_bounds__(64) void latent_heads_merge_kernel(LatentArgs a) {
    const int lane = threadIdx.x, n32 = lane & 31, h = lane >> 5;
    const int wave = blockIdx.x & 3, unit = blockIdx.x >> 2, vb = blockIdx.y >> 2, hb = blockIdx.y & 3;
    const int r = unit / a.tiles, group = unit - r * a.tiles;
    const int H = a.heads;
    const int j = group * kHeadsRows + hb * 32 + n32, col = j / H, head = j - col * H;
    int count = a.columns;
    if (a.counts) count = min(a.counts[r], a.columns);
    if (col >= count) return;
    const int64_t first64 = a.firsts[r];
    const int first = (int)(first64 < 0 ? 0 : (first64 > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : first64));
    const int n_keys = min(first + col + 1, a.max_keys);
    const int n_pieces = (n_keys + a.piece - 1) / a.piece;
    const int np = min(a.parts, n_pieces);
    const int64_t index = ((int64_t)((int64_t)r * a.columns + col) * H + head) * a.parts;
    const float* slab = a.po + ((int64_t)unit * a.parts * 4 + wave) * (int64_t)(kHeadsRows * R / 4) + (vb * 4 + hb) * 1024 + lane * 4;
    float M = -INFINITY, L = 0.0f, acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
    constexpr int AHEAD = 4;      // partitions requested together (past the last one the last again, so every load is issued)
    for (int b0 = 0; b0 < np; b0 += AHEAD) {
        float pm[AHEAD], pl[AHEAD];
        float4 po[AHEAD][4];
#pragma unroll
        for (int k = 0; k < AHEAD; ++k) {
            const int b = min(b0 + k, np - 1);
            pm[k] = a.pm[index + b], pl[k] = a.pl[index + b];
#pragma unroll
            for (int v4 = 0; v4 < 4; ++v4)
                po[k][v4] = *reinterpret_cast<const float4*>(slab + (int64_t)b * 4 * (kHeadsRows * R / 4) + v4 * 256);
        }
#pragma unroll
        for (int k = 0; k < AHEAD; ++k) {
            if (b0 + k < np) {
                const Fold f = fold(M, L, pm[k], pl[k]);
#pragma unroll
                for (int v4 = 0; v4 < 4; ++v4) {
                    acc[4 * v4] = __builtin_fmaf(acc[4 * v4], f.keep, po[k][v4].x * f.take);
                    acc[4 * v4 + 1] = __builtin_fmaf(acc[4 * v4 + 1], f.keep, po[k][v4].y * f.take);
                    acc[4 * v4 + 2] = __builtin_fmaf(acc[4 * v4 + 2], f.keep, po[k][v4].z * f.take);
                    acc[4 * v4 + 3] = __builtin_fmaf(acc[4 * v4 + 3], f.keep, po[k][v4].w * f.take);
                }
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
        for (int i = 0; i < 16; ++i) acc[i] *= keep;
        M = top;
    }
    const int64_t token = (int64_t)a.starts[r] + col;
    const float inv = L > 0.0f ? 1.0f / L : 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i)
        store_out(a.out, a.out_dtype, token * a.o_st + (int64_t)head * a.o_sh + wave * 128 + vb * 32 + 8 * (i / 4) + 4 * h + i % 4, acc[i] * inv);
    if (a.lse && wave == 0 && vb == 0 && h == 0) a.lse[token * a.heads + head] = (L > 0.0f || L != L) ? (M + __builtin_log2f(L)) * kLn2 : -INFINITY;
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

// -- the shapes whose rows do not fill the tiles above (ranks 16 and 32, a rotary width of 16) -----------------------------
// A wavefront serves one query row (a batch row's column and head) over pieces b, b + parts, ... of the positions it
// sees, 64 positions a step with a lane a position: the lane reads its position's whole cache row for the score (the
// query's values wait in LDS as FP32), the step's softmax runs over the wavefront, and for the values the lanes turn
// to the row's dims (lane i: values 2 i, 2 i + 1 of every 128) while the positions' probabilities and slots go round by
// shuffle. No matrix pipe and every cache row read twice (the second time from the caches): these shapes are served,
// not tuned. The partials have the layout and the meaning of the kernels' above.
template <bool F16, bool FP8>
__global__ __launch_bounds__(256) void latent_plain_kernel(LatentArgs a, int R, int P, int groups) {
    constexpr int EB = FP8 ? 1 : 2;
    __shared__ float s_q[4][1024 + 256];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int W = R + P;
    const int64_t pair = blockIdx.x / groups;
    const int group = (int)(blockIdx.x - pair * groups);
    const int r = (int)(pair / a.gy), b = (int)(pair % a.gy);
    const int H = a.heads;
    int count = a.columns;
    if (a.counts) count = min(a.counts[r], a.columns);
    const int jq = group * 4 + wave, colq = jq / H, headq = jq - colq * H;
    const bool liveq = colq < count;
    if (liveq) {
        const uint8_t* q = a.q + ((int64_t)(a.starts[r] + colq) * a.q_st + (int64_t)headq * a.q_sh) * 2;
        for (int e = lane * 2; e < W; e += 128) {
            const uint32_t w = *reinterpret_cast<const uint32_t*>(q + e * 2);
            s_q[wave][e] = F16 ? f16_lo(w) : bf16_lo(w);
            s_q[wave][e + 1] = F16 ? f16_hi(w) : bf16_hi(w);
        }
    }
    __syncthreads();
    if (!liveq) return;
    const int64_t first64 = a.firsts[r];
    const int first = (int)(first64 < 0 ? 0 : (first64 > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : first64));
    const int n_keys = min(first + colq + 1, a.max_keys);      // the positions this query row sees
    const int n_pieces = (n_keys + a.piece - 1) / a.piece;
    if (b >= n_pieces) return;
    const int64_t trow = (int64_t)a.rows[(int64_t)r * a.rows_step] * a.tab_stride;
    const float* query = s_q[wave];

    float m = -INFINITY, l = 0.0f, acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
    for (int pi = b; pi < n_pieces; pi += a.parts) {
        const int piece_end = min((pi + 1) * a.piece, n_keys);      // (partitions * piece is bounded by the launch)
        for (int base = pi * a.piece; base < piece_end; base += 64) {
            const bool seen = base + lane < piece_end;
            const int n = seen ? base + lane : piece_end - 1;
            const int pidx = (int)div32(a.page_div, (uint32_t)n);
            const int entry = a.tables[trow + (pidx < a.tab_width ? pidx : a.tab_width - 1)];
            const int64_t slot = (int64_t)entry * a.page + (n - pidx * a.page);
            const uint8_t* row = a.cache + slot * (W * EB);
            float s0 = 1.0f, s1 = 1.0f;
            if constexpr (FP8) {
                const float* sc = a.scales + slot * a.scales_per_row;
                s0 = sc[0], s1 = a.scales_per_row > 1 ? sc[1] : s0;
            }
            float dots[2] = {0.0f, 0.0f};      // the latent's products, then the rotary key's
#pragma unroll
            for (int part = 0; part < 2; ++part) {
                const int e0 = part ? R : 0, e1 = part ? W : R;
                float dot = 0.0f;
                for (int e = e0; e < e1; e += 16 / EB) {
                    const u32x4 w = *reinterpret_cast<const u32x4*>(row + e * EB);
                    const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        if constexpr (FP8) {
                            const f32x2 lo = e4m3_pair<false>(ws[k]), hi = e4m3_pair<true>(ws[k]);
                            dot = __builtin_fmaf(lo.x, query[e + 4 * k], dot);
                            dot = __builtin_fmaf(lo.y, query[e + 4 * k + 1], dot);
                            dot = __builtin_fmaf(hi.x, query[e + 4 * k + 2], dot);
                            dot = __builtin_fmaf(hi.y, query[e + 4 * k + 3], dot);
                        } else {
                            dot = __builtin_fmaf(F16 ? f16_lo(ws[k]) : bf16_lo(ws[k]), query[e + 2 * k], dot);
                            dot = __builtin_fmaf(F16 ? f16_hi(ws[k]) : bf16_hi(ws[k]), query[e + 2 * k + 1], dot);
                        }
                    }
                }
                dots[part] = dot;
            }
            float x = (FP8 ? __builtin_fmaf(dots[0], s0, dots[1] * s1) : dots[0] + dots[1]) * a.sscale;
            x = seen ? x : -INFINITY;
            const float m_new = __builtin_fmaxf(m, group_max<64>(x));
            const float sub = m_new == -INFINITY ? 0.0f : m_new;
            const float alpha = exp2_fast(m - sub);
            float p = exp2_fast(x - sub);
            l = __builtin_fmaf(l, alpha, group_sum<64>(p));
            m = m_new;
            if constexpr (FP8) p *= s0;      // a value is its code times its position's latent scale
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] *= alpha;
            const int lo = (int)(uint32_t)slot, hi = (int)(slot >> 32);
            const int live = min(64, piece_end - base);
            for (int j = 0; j < live; ++j) {
                const float pj = __shfl(p, j);
                const int64_t at = ((int64_t)__shfl(hi, j) << 32) | (uint32_t)__shfl(lo, j);
                const uint8_t* values = a.cache + at * (W * EB) + lane * 2 * EB;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (i * 128 + lane * 2 < R) {
                        float v0, v1;
                        if constexpr (FP8) {
                            const f32x2 v = e4m3_pair<false>(*reinterpret_cast<const uint16_t*>(values + i * 128));
                            v0 = v.x, v1 = v.y;
                        } else {
                            const uint32_t w = *reinterpret_cast<const uint32_t*>(values + i * 256);
                            v0 = F16 ? f16_lo(w) : bf16_lo(w), v1 = F16 ? f16_hi(w) : bf16_hi(w);
                        }
                        acc[2 * i] = __builtin_fmaf(pj, v0, acc[2 * i]);
                        acc[2 * i + 1] = __builtin_fmaf(pj, v1, acc[2 * i + 1]);
                    }
                }
            }
        }
    }
    const int64_t index = ((int64_t)((int64_t)r * a.columns + colq) * H + headq) * a.parts + b;
#pragma unroll
    for (int i = 0; i < 8; ++i)
        if (i * 128 + lane * 2 < R)
            *reinterpret_cast<f32x2*>(a.po + index * R + i * 128 + lane * 2) = f32x2{acc[2 * i], acc[2 * i + 1]};
    if (lane == 0) a.pm[index] = m, a.pl[index] = l;
}

// Its merge: latent_merge_kernel with the rank at run time (a thread: values t, t + 64, ... one after another).
__global__ __launch_bounds__(64) void latent_plain_merge_kernel(LatentArgs a, int R) {
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
    const int64_t token = (int64_t)a.starts[r] + col;
    for (int d = threadIdx.x; d < R; d += 64) {
        float M = -INFINITY, L = 0.0f, acc = 0.0f;
        for (int b = 0; b < np; ++b) {
            const Fold f = fold(M, L, a.pm[index + b], a.pl[index + b]);
            acc = __builtin_fmaf(acc, f.keep, a.po[(index + b) * R + d] * f.take);
            M = f.m, L = f.l;
        }
        if (a.sinks) {      // one more position with no value
            const float sink = a.sinks[head] * kLog2e;
            const float top = __builtin_fmaxf(M, sink);
            const float sub = top == -INFINITY ? 0.0f : top;
            const float keep = exp2_fast(M - sub);
            L = __builtin_fmaf(L, keep, exp2_fast(sink - sub));
            acc *= keep;
            M = top;
        }
        const float inv = L > 0.0f ? 1.0f / L : 0.0f;
        store_out(a.out, a.out_dtype, token * a.o_st + (int64_t)head * a.o_sh + d, acc * inv);
        if (a.lse && d == 0) a.lse[token * a.heads + head] = (L > 0.0f || L != L) ? (M + __builtin_log2f(L)) * kLn2 : -INFINITY;
    }
}

int launch_plain(const LatentArgs& a, int R, int P, bool f16, bool fp8, int phases, hipStream_t stream) {
    if (phases != 2) {
        const int groups = (a.columns * a.heads + 3) / 4;
        const int64_t blocks = a.pairs * groups;
        if (blocks > 0x7fffffff) return CRIT_PKV_E_GEOMETRY;
        const dim3 grid((unsigned)blocks);
        if (fp8) {
            if (f16) hipLaunchKernelGGL((latent_plain_kernel<true, true>), grid, dim3(256), 0, stream, a, R, P, groups);
            else hipLaunchKernelGGL((latent_plain_kernel<false, true>), grid, dim3(256), 0, stream, a, R, P, groups);
        } else {
            if (f16) hipLaunchKernelGGL((latent_plain_kernel<true, false>), grid, dim3(256), 0, stream, a, R, P, groups);
            else hipLaunchKernelGGL((latent_plain_kernel<false, false>), grid, dim3(256), 0, stream, a, R, P, groups);
        }
        const int bad = hip_code(hipGetLastError());
        if (bad) return bad;
    }
    if (phases != 1) {
        hipLaunchKernelGGL(latent_plain_merge_kernel, dim3((unsigned)(a.n_rows * a.columns), (unsigned)a.heads), dim3(64), 0, stream, a, R);
        return hip_code(hipGetLastError());
    }
    return 0;
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

// Which launches the many-heads kernel serves: caches of the one shape it is built for with pages of a multiple of 16
// positions, where the caller asks for it (any number of heads: a tile of 128 rows is then 128 / heads columns of
// a window, which is how a prompt chunk of few heads fills it) or, left to the library, where the heads come in 128s.
// (Nothing else decides, the batch least of all: a token's bits follow the kernel that reads it.)
template <int R, int P>
bool many_heads(const LatentArgs& a, bool fp8) {
    if (!(R == 512 && P == 64 && a.page % 16 == 0)) return false;
    return a.tile_rows == kHeadsRows || (a.tile_rows == 0 && a.heads % kHeadsRows == 0);
}

template <int R, int P>
int launch_shape(const LatentArgs& a, bool f16, bool fp8, int phases, hipStream_t stream) {
    if constexpr (R == 512 && P == 64) {
        if (many_heads<R, P>(a, fp8)) {
            LatentArgs u = a;
            u.tiles = (a.columns * a.heads + kHeadsRows - 1) / kHeadsRows;
            const int64_t blocks = (a.n_rows >= kRowsToAnXcd ? (int64_t)((a.n_rows + 7) / 8) * 8 * a.gy : (u.pairs + 7) / 8 * 8) * u.tiles;
            const int64_t merges = (int64_t)a.n_rows * u.tiles * 4;
            if (blocks > 0x7fffffff || merges > 0x7fffffff) return CRIT_PKV_E_GEOMETRY;
            if (phases != 2) {
                if (fp8) {
                    if (f16) hipLaunchKernelGGL((latent_heads_kernel<R, P, true, true>), dim3((unsigned)blocks), dim3(256), 0, stream, u);
                    else hipLaunchKernelGGL((latent_heads_kernel<R, P, false, true>), dim3((unsigned)blocks), dim3(256), 0, stream, u);
                } else {
                    if (f16) hipLaunchKernelGGL((latent_heads_kernel<R, P, true, false>), dim3((unsigned)blocks), dim3(256), 0, stream, u);
                    else hipLaunchKernelGGL((latent_heads_kernel<R, P, false, false>), dim3((unsigned)blocks), dim3(256), 0, stream, u);
                }
                const int bad = hip_code(hipGetLastError());
                if (bad) return bad;
            }
            if (phases != 1) {
                hipLaunchKernelGGL((latent_heads_merge_kernel<R>), dim3((unsigned)merges, 16), dim3(64), 0, stream, u);
                return hip_code(hipGetLastError());
            }
            return 0;
        }
    }
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
    a.tile_rows = p->tile_rows;
    if (p->tile_rows != 0 && p->tile_rows != 16 && p->tile_rows != kHeadsRows) return CRIT_PKV_E_GEOMETRY;
    if (p->tile_rows == kHeadsRows && !(p->rank == 512 && p->rope == 64 && p->page % 16 == 0)) return CRIT_PKV_E_GEOMETRY;
    a.tiles = (p->columns * p->heads + 15) / 16;
    const int64_t table_keys = (int64_t)p->table_width * p->page;
    a.max_keys = (int)(table_keys < 0x3fffffff ? table_keys : 0x3fffffff);
    if ((int64_t)p->partitions * p->piece > 0x3fffffff) return CRIT_PKV_E_WORKSPACE;
    const int64_t live_parts = ((int64_t)a.max_keys + p->piece - 1) / p->piece;
    a.gy = (int)(live_parts < p->partitions ? live_parts : p->partitions);
    a.pairs = (int64_t)p->n_rows * a.gy;
    const bool f16 = p->q_dtype == CRIT_PKV_F16;
#define PKV_LATENT(RANK, ROPE) \
    if (p->rank == RANK && p->rope == ROPE) return launch_shape<RANK, ROPE>(a, f16, fp8, p->phases , stream);
    PKV_LATENT(512, 64) PKV_LATENT(256, 64) PKV_LATENT(128, 64) PKV_LATENT(128, 32) PKV_LATENT(64, 64) PKV_LATENT(64, 32)
    PKV_LATENT(1024, 64) PKV_LATENT(512, 128)
    PKV_LATENT(1024, 32) PKV_LATENT(1024, 128) PKV_LATENT(1024, 256) PKV_LATENT(512, 32) PKV_LATENT(512, 256) PKV_LATENT(256, 32)
    PKV_LATENT(256, 128) PKV_LATENT(256, 256) PKV_LATENT(128, 128) PKV_LATENT(128, 256) PKV_LATENT(64, 128) PKV_LATENT(64, 256)
#undef PKV_LATENT
    const auto power_of_two = [](int x, int lo, int hi) { return x >= lo && x <= hi && (x & (x - 1)) == 0; };
    if (power_of_two(p->rank, 16, 1024) && power_of_two(p->rope, 16, 256) && p->tile_rows != kHeadsRows)
        return launch_plain(a, p->rank, p->rope, f16, fp8, p->phases, stream);
    return CRIT_PKV_E_GEOMETRY;
}

}   // namespace pkv
