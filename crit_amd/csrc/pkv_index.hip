// Sparse index selection for gfx950: every query token's score over the compressed keys it may see, and the positions
// of its k best, which a block-sparse attention then reads. What the reference's sparse-indexer kernels module computes
// (kernels/techniques/attention/sparse-indexer/torch-ext/sparse_indexer/__init__.py:83-139, _kernels.py; the operation:
// inference/attention-state/code/sparse_index.py):
//   score[t][s] = sum_h weights[t][h] * scale * max(0, q[t][h] . keys[s])   for s < ends[t], -inf at or past it
//   picked[t]   = the positions of the k largest scores below ends[t], ascending, then -1; ties to the lower position,
//                 a NaN below every number
//
// Scores. A token's queries stay in registers as A operands of v_mfma_f32_16x16x32 (a lane: one head of a tile of 16,
// 8 adjacent values per k-step), a tile of 16 keys is the B operand (a lane: one key), so a lane is left 4 heads'
// products with one key: ReLU, the head's factor, the lane's heads added in order, the tiles of heads in order, then
// the four quarters of the wavefront as (0 + 1) + (2 + 3). That order is the same in both kernels, so a token's bits
// are its own: not its neighbours', not the launch's shape.
//   index_scores_kernel: a workgroup is one token and a block of keys, its four wavefronts take tiles of 16 keys in
//     turn and load them where they lie (from their slots where the keys are read in place): calls of few tokens.
//   index_scores_tokens_kernel: a workgroup is 4 or 8 tokens (one or two a wavefront) and a block of keys; 64 keys a
//     step go through LDS once for all of them (two buffers, one barrier a step, the next step's loads in flight
//     under the products), so the keys cross the L2 once per 4 or 8 tokens.
//
// Top-k. The scores map to 32-bit keys that order as the rule does (NaN lowest, -0 = +0); a radix select from the top
// finds the k-th key and how many of its equals are taken; then the positions of everything above the k-th key and of
// its first equals are written in order: ascending by construction.
//   index_topk_runs_kernel: a workgroup holds a row (or a slice of one) in registers, a thread a run of consecutive
//     positions: digits of 11, 11 and 10 bits, the places of a thread's picks from its own counts and one scan.
//   index_topk_kernel: rows no workgroup can hold stream through 8-bit digits, a workgroup a row.
// Calls of few tokens over many positions select in slices (the k best of each, positions and scores) and then among
// the slices' picks: a token's k best are among its slices', in the same order.
#include "pkv_attend_mfma.hpp"
#include "pkv_launch.hpp"

namespace pkv {
namespace {

struct ScoreArgs {
    const uint8_t* q;
    const uint8_t* keys;
    const float* key_scales;
    const float* weights;
    const int32_t* ends;
    const void* slots;
    float* out;
    int64_t q_st, q_sh, key_stride, w_stride, out_stride, slots_stride;
    int tokens, n, group, heads, slots_are_64, block;
    float scale;
};

// One token's queries: qa[ht][ks] the lane's A operand (head ht * 16 + li, 8 adjacent values per k-step), heads past
// the last as zeros. Which 8 values: the ones the lane's key operand holds at that step. 16-bit keys: values
// ks * 32 + 8 g .. + 7 (a lane loads 16 bytes of its key a step). E4M3 keys: a lane loads 16 bytes, 16 values, for a
// pair of steps, so steps 2 j and 2 j + 1 take values 64 j + 16 g .. + 7 and + 8 .. + 15 (a sum over the values in
// another order; both kernels use the same one).
template <int HT, int KS>
struct TokenQ {
    u32x4 qa[HT][KS];
};

// Where in a head's row of 16-bit queries (in bytes) the lane's operand of step ks starts.
template <bool FP8>
PKV_DEV constexpr int q_offset(int ks, int g) {
    return FP8 ? (ks >> 1) * 128 + g * 32 + (ks & 1) * 16 : ks * 64 + g * 16;
}

template <bool FP8, int HT, int KS>
PKV_DEV void load_token(const ScoreArgs& a, int t, int g, int li, TokenQ<HT, KS>& q) {
#pragma unroll
    for (int ht = 0; ht < HT; ++ht) {
        const int h = ht * 16 + li;
        const uint8_t* row = a.q + ((int64_t)t * a.q_st + (int64_t)h * a.q_sh) * 2;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4 w = {0u, 0u, 0u, 0u};
            if (h < a.heads) w = *reinterpret_cast<const u32x4*>(row + q_offset<FP8>(ks, g));
            q.qa[ht][ks] = w;
        }
    }
}

// The factor of head h of token t (0 past the last head).
PKV_DEV float head_factor(const ScoreArgs& a, int t, int h) {
    return h < a.heads ? a.weights[(int64_t)t * a.w_stride + h] * a.scale : 0.0f;
}

// A key's lane operand from what was loaded: 16-bit values as they are, E4M3 codes as their 16-bit values (exact).
template <bool F16, bool FP8>
PKV_DEV u32x4 key_operand(u32x4 raw16, u32x2 raw8) {
    if constexpr (FP8) {
        const f32x2 a0 = e4m3_pair<false>(raw8.x), a1 = e4m3_pair<true>(raw8.x), a2 = e4m3_pair<false>(raw8.y), a3 = e4m3_pair<true>(raw8.y);
        return u32x4{pair16<F16>(a0.x, a0.y), pair16<F16>(a1.x, a1.y), pair16<F16>(a2.x, a2.y), pair16<F16>(a3.x, a3.y)};
    } else {
        return raw16;
    }
}

// max(x, 0) as one instruction: the bits of a float order as a signed integer's do where it is positive, and every
// negative float (and -0) is a negative integer (fmaxf comes with a second instruction that quiets a signalling NaN).
PKV_DEV float relu(float x) { return u2f((uint32_t)max((int)f2u(x), 0)); }

// A token's score with the lane's key (the tile's key li), the same bits in the four lanes of the key: f(ht) gives the
// factors of heads ht * 16 + 4 g .. + 3.
template <bool F16, int HT, int KS, typename Factors>
PKV_DEV float tile_score(const TokenQ<HT, KS>& q, const u32x4 (&kb)[KS], Factors&& f) {
    f32x4 acc[HT];
#pragma unroll
    for (int ht = 0; ht < HT; ++ht) acc[ht] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int ht = 0; ht < HT; ++ht) acc[ht] = mfma_k32<F16>(q.qa[ht][ks], kb[ks], acc[ht]);
    float total = 0.0f;
#pragma unroll
    for (int ht = 0; ht < HT; ++ht) {
        const f32x4 w = f(ht);
#pragma unroll
        for (int i = 0; i < 4; ++i) total = __builtin_fmaf(relu(acc[ht][i]), w[i], total);      // (one rounding a head)
    }
    return sum_across_quarters(total);
}

PKV_DEV int64_t slot_of(const ScoreArgs& a, int64_t srow, int key) {
    if (!a.slots) return key;
    return a.slots_are_64 ? reinterpret_cast<const int64_t*>(a.slots)[srow + key] : (int64_t) reinterpret_cast<const int32_t*>(a.slots)[srow + key];
}

template <bool F16, bool FP8, int HT, int KS, int PD>
__global__ __launch_bounds__(256) void index_scores_kernel(ScoreArgs a) {
    constexpr int QROWB = KS * 64 + (HT * KS == 64 ? 0 : 16);      // a head's row in LDS (padded where that keeps it within 64 KB)
    __shared__ __align__(16) uint8_t s_q[HT * 16 * QROWB];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, g = lane >> 4, li = lane & 15;
    const int t = blockIdx.y;
    // the token's queries: loaded once a workgroup, then each wavefront's operands from LDS (heads past the last: zeros)
    for (int i = tid; i < HT * 16 * KS * 4; i += 256) {
        const int h = i / (KS * 4), c = i % (KS * 4);
        u32x4 w = {0u, 0u, 0u, 0u};
        if (h < a.heads) w = *reinterpret_cast<const u32x4*>(a.q + ((int64_t)t * a.q_st + (int64_t)h * a.q_sh) * 2 + c * 16);
        *reinterpret_cast<u32x4*>(s_q + h * QROWB + c * 16) = w;
    }
    f32x4 fac[HT];
#pragma unroll
    for (int ht = 0; ht < HT; ++ht)
#pragma unroll
        for (int i = 0; i < 4; ++i) fac[ht][i] = head_factor(a, t, ht * 16 + 4 * g + i);
    const int end = min(max(a.ends[t], 0), a.n);
    const int64_t srow = (int64_t)(t / a.group) * a.slots_stride;
    const int first = blockIdx.x * a.block;
    const int last = min(first + a.block, a.n);
    float* out = a.out + (int64_t)t * a.out_stride;
    constexpr int LD = FP8 ? KS / 2 : KS;      // 16-byte loads a key a lane
    // The wavefront's tiles (wave, wave + 4, ... of the block's tiles of 16 keys) that hold a key the token sees go
    // through a pipeline of PD stages: a tile's key row is requested PD tiles before its products and its slot is
    // looked up PD tiles before that (loads return in order: a slot wanted sooner would wait for every row requested
    // after it), and every load of the loop is issued whether or not its tile exists (past the last one it repeats
    // the last), so the waits are exact counts. Tiles wholly past the token's end are only written. PD: 3 where a
    // wavefront has many tiles (the launcher's rule), else 1.
    const int seen_last = min(last, end);      // keys below it are seen
    const int n_tiles = seen_last > first + wave * 16 ? (seen_last - first - wave * 16 + 63) / 64 : 0;
    auto tile_k0 = [&](int i) { return first + (wave + 4 * i) * 16; };
    auto slot_load = [&](int i) -> int64_t {
        const int ii = i < n_tiles ? i : n_tiles - 1;
        return slot_of(a, srow, min(tile_k0(ii) + li, a.n - 1));
    };
    u32x4 held[PD][LD];
    int64_t at_s[PD];
    float ksc[PD];
    auto row_load = [&](auto sc, int64_t at) __attribute__((always_inline)) {
        constexpr int st = decltype(sc)::value;
        at_s[st] = at;
        const uint8_t* krow = a.keys + at * a.key_stride * (FP8 ? 1 : 2) + g * 16;
#pragma unroll
        for (int j = 0; j < LD; ++j) held[st][j] = *reinterpret_cast<const u32x4*>(krow + j * 64);
        if constexpr (FP8) ksc[st] = a.key_scales[at];
    };
    int64_t ahead[PD];      // the slots of the tiles PD past the ones whose rows are in flight
    if (n_tiles > 0) {
        static_for<PD>([&](auto sc) __attribute__((always_inline)) { row_load(sc, slot_load(decltype(sc)::value)); });
        static_for<PD>([&](auto sc) __attribute__((always_inline)) { ahead[decltype(sc)::value] = slot_load(PD + decltype(sc)::value); });
    }
    __syncthreads();
    TokenQ<HT, KS> q;
#pragma unroll
    for (int ht = 0; ht < HT; ++ht)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) q.qa[ht][ks] = *reinterpret_cast<const u32x4*>(s_q + (ht * 16 + li) * QROWB + q_offset<FP8>(ks, g));
    for (int i = 0; i < n_tiles; i += PD) {
        static_for<PD>([&](auto sc) __attribute__((always_inline)) {
            constexpr int st = decltype(sc)::value;
            const int ii = i + st;
            u32x4 kb[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                if constexpr (FP8) {
                    const u32x4 w = held[st][ks >> 1];
                    kb[ks] = key_operand<F16, true>(u32x4{}, (ks & 1) ? u32x2{w.z, w.w} : u32x2{w.x, w.y});
                } else {
                    kb[ks] = held[st][ks];
                }
            }
            float scale_of_key = 1.0f;
            if constexpr (FP8) scale_of_key = ksc[st];
            if (PD > 1 || ii + PD < n_tiles) {      // (one stage: only the tiles there are; more: every load, see above)
                row_load(sc, ahead[st]);            // tile ii + PD's row (a tile past the last: the last one's again)
                ahead[st] = slot_load(ii + 2 * PD);
            }
            float v = tile_score<F16>(q, kb, [&](int ht) { return fac[ht]; });
            if constexpr (FP8) v *= scale_of_key;
            const int kk = tile_k0(ii) + li;
            if (ii < n_tiles && g == 0 && kk < last) out[kk] = kk < end ? v : -INFINITY;
        });
    }
    // the wavefront's tiles wholly at or past the token's end
    for (int k0 = tile_k0(n_tiles); k0 < last; k0 += 64)
        if (g == 0 && k0 + li < last) out[k0 + li] = -INFINITY;
}

template <bool F16, bool FP8, int HT, int KS, int TW>
__global__ __launch_bounds__(256, HT * KS * TW <= 32 ? 2 : 1) void index_scores_tokens_kernel(ScoreArgs a) {
    constexpr int E = FP8 ? 1 : 2;
    constexpr int ROWB = KS * 32 * E + 16;            // a key's row in LDS
    constexpr int CH = KS * 32 * E / 16;              // its 16-byte pieces
    constexpr int PER = 64 * CH / 256;                // pieces a thread stages a step
    constexpr int HP = HT * 16;
    extern __shared__ __align__(16) uint8_t s_mem[];  // the heads' factors [4 TW][HP], then two buffers of 64 key rows
    float* s_f = reinterpret_cast<float*>(s_mem);
    uint8_t* s_k = s_mem + 4 * TW * HP * 4;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, g = lane >> 4, li = lane & 15;
    const int wg_first = blockIdx.y * (4 * TW);
    TokenQ<HT, KS> q[TW];
    int ends[TW];
    bool live[TW];
    int wave_end = 0;
#pragma unroll
    for (int j = 0; j < TW; ++j) {
        const int t = wg_first + wave * TW + j;
        live[j] = t < a.tokens;
        const int tt = live[j] ? t : a.tokens - 1;
        load_token<FP8>(a, tt, g, li, q[j]);
        ends[j] = live[j] ? min(max(a.ends[tt], 0), a.n) : 0;
        wave_end = max(wave_end, ends[j]);
    }
    for (int i = tid; i < 4 * TW * HP; i += 256) {
        const int t = wg_first + i / HP;
        s_f[i] = t < a.tokens ? head_factor(a, t, i % HP) : 0.0f;
    }
    const int64_t srow = (int64_t)(wg_first / a.group) * a.slots_stride;      // (a workgroup's tokens are of one group)
    const int first = blockIdx.x * a.block;
    const int last = min(first + a.block, a.n);
    u32x4 held[PER];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int c = tid + 256 * j;
            const int64_t at = slot_of(a, srow, min(k0 + c / CH, a.n - 1));
            held[j] = *reinterpret_cast<const u32x4*>(a.keys + at * a.key_stride * E + (c % CH) * 16);
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int c = tid + 256 * j;
            *reinterpret_cast<u32x4*>(s_k + buf * (64 * ROWB) + (c / CH) * ROWB + (c % CH) * 16) = held[j];
        }
    };
    fetch(first);
    int buf = 0;
    for (int k0 = first; k0 < last; k0 += 64, buf ^= 1) {
        stage(buf);
        lds_barrier();      // (one a step: a buffer is written again two steps on, past the barrier every wavefront reaches after its reads)
        if (k0 + 64 < last) fetch(k0 + 64);
        const int kk = k0 + lane;
        float mine[TW];
#pragma unroll
        for (int j = 0; j < TW; ++j) mine[j] = 0.0f;
        if (k0 < wave_end) {
            f32x4 fac[TW][HT];
#pragma unroll
            for (int j = 0; j < TW; ++j)
#pragma unroll
                for (int ht = 0; ht < HT; ++ht) fac[j][ht] = *reinterpret_cast<const f32x4*>(s_f + (wave * TW + j) * HP + ht * 16 + 4 * g);
#pragma unroll
            for (int T = 0; T < 4; ++T) {
                const uint8_t* krow = s_k + buf * (64 * ROWB) + (T * 16 + li) * ROWB + g * 16;
                u32x4 kb[KS];
                if constexpr (FP8) {
#pragma unroll
                    for (int j = 0; j < KS / 2; ++j) {
                        const u32x4 w = *reinterpret_cast<const u32x4*>(krow + j * 64);
                        kb[2 * j] = key_operand<F16, true>(u32x4{}, u32x2{w.x, w.y});
                        kb[2 * j + 1] = key_operand<F16, true>(u32x4{}, u32x2{w.z, w.w});
                    }
                } else {
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) kb[ks] = *reinterpret_cast<const u32x4*>(krow + ks * 64);
                }
#pragma unroll
                for (int j = 0; j < TW; ++j) {
                    const float v = tile_score<F16>(q[j], kb, [&](int ht) { return fac[j][ht]; });
                    if (g == T) mine[j] = v;      // the quarter g keeps tile g: a lane's key is k0 + lane
                }
            }
        }
        float key_scale = 1.0f;
        if constexpr (FP8) key_scale = a.key_scales[slot_of(a, srow, min(kk, a.n - 1))];
#pragma unroll
        for (int j = 0; j < TW; ++j)
            if (live[j] && kk < last)
                a.out[(int64_t)(wg_first + wave * TW + j) * a.out_stride + kk] = kk < ends[j] ? mine[j] * key_scale : -INFINITY;
    }
}

struct TopkArgs {
    const float* s;          // scores [tokens][s_stride]; the candidates' where LEVEL is 2
    const int32_t* pos;      // the candidates' positions [tokens][s_stride] (LEVEL 2)
    const int32_t* ends;
    int32_t* out;
    float* out_scores;       // the picks' scores beside their positions (LEVEL 1)
    int64_t s_stride, out_stride;
    int tokens, n, k, width, parts;
};

// The key a score is ranked by: larger first; -0 and +0 the same; -inf below every finite; a NaN below everything.
PKV_DEV uint32_t rank_key(float x) {
    if (x != x) return 0u;
    uint32_t u = f2u(x == 0.0f ? 0.0f : x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// A score that ranks as `key` does (the score itself but for -0, which comes back +0, and a NaN's payload).
PKV_DEV float score_of_key(uint32_t key) {
    if (key == 0u) return u2f(0x7fc00000u);
    return u2f((key & 0x80000000u) ? (key ^ 0x80000000u) : ~key);
}

// LEVEL 0: a token's row, to its picks. 1: a slice of its row (blockIdx.y), to the slice's candidates (positions and
// scores, [parts][k] a token). 2: a token's candidates (those with a position), to its picks.
template <int LEVEL>
__global__ __launch_bounds__(256) void index_topk_kernel(TopkArgs a) {
    __shared__ unsigned s_hist[256 * 16];
    __shared__ unsigned s_wave[4];
    __shared__ unsigned s_pick[2];
    __shared__ int s_cnt[4][2];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int t = blockIdx.x, part = LEVEL == 1 ? blockIdx.y : 0;
    const int end = min(max(a.ends[t], 0), a.n);
    const int k = a.k;
    const float* row = a.s + (int64_t)t * a.s_stride;
    const int32_t* pos = LEVEL == 2 ? a.pos + (int64_t)t * a.s_stride : nullptr;
    int32_t* out = a.out + (int64_t)t * a.out_stride + (int64_t)part * k;
    float* out_scores = LEVEL == 1 ? a.out_scores + (int64_t)t * a.out_stride + (int64_t)part * k : nullptr;
    int lo = 0, m, valid;      // the elements lo .. lo + m - 1 of the row, `valid` of them candidates
    if constexpr (LEVEL == 2) {
        m = a.parts * k, valid = 0;
        for (int p = 0; p < a.parts; ++p) valid += min(max(min(end - p * a.width, a.width), 0), k);
    } else {
        lo = LEVEL == 1 ? part * a.width : 0;
        m = max(min(LEVEL == 1 ? a.width : a.n, end - lo), 0), valid = m;
    }
    row += lo;
    auto take = [&](int i, float& x) -> bool {      // element i: its score; whether it is a candidate
        if constexpr (LEVEL == 2) {
            if (pos[i] < 0) return false;
        }
        x = row[i];
        return true;
    };
    const bool all = valid <= k;      // everything is picked
    uint32_t prefix = 0u;
    unsigned want = 0u;               // of the keys equal to the k-th, the `want` first are taken
    if (!all) {
        // radix select: the k-th largest key, 8 bits at a time from the top
        uint32_t mask = 0u;
        want = (unsigned)k;
        for (int shift = 24; shift >= 0; shift -= 8) {
#pragma unroll
            for (int j = 0; j < 16; ++j) s_hist[tid + 256 * j] = 0u;
            __syncthreads();
            for (int i0 = 0; i0 < m; i0 += 1024) {
                float x[4];
                bool ok[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int i = i0 + j * 256 + tid;
                    x[j] = 0.0f;
                    ok[j] = i < m && take(i, x[j]);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t key = rank_key(x[j]);
                    if (ok[j] && (key & mask) == prefix) atomicAdd(&s_hist[((key >> shift) & 255u) * 16 + (lane & 15)], 1u);
                }
            }
            __syncthreads();
            // thread tid: bin 255 - tid; the count of keys in it and in the bins above it
            const int bin = 255 - tid;
            unsigned h = 0u;
#pragma unroll
            for (int j = 0; j < 16; ++j) h += s_hist[bin * 16 + j];
            unsigned incl = wave_inclusive_sum(h);
            if (lane == 63) s_wave[wave] = incl;
            __syncthreads();
            for (int w = 0; w < wave; ++w) incl += s_wave[w];
            if (incl >= want && incl - h < want) s_pick[0] = (unsigned)bin, s_pick[1] = want - (incl - h);
            __syncthreads();
            prefix |= s_pick[0] << shift;
            mask |= 255u << shift;
            want = s_pick[1];
        }
    }
    // In position order: everything above the k-th key, and its first `want` equals. A wavefront takes a quarter of the
    // elements: what it will write first, then the writes.
    const int per = (m + 255) / 256 * 64;
    const int w_lo = min(wave * per, m), w_hi = min(w_lo + per, m);
    const unsigned long long below = (1ull << lane) - 1ull;
    int n_above = 0, n_equal = 0;
    for (int i0 = w_lo; i0 < w_hi; i0 += 64) {
        const int i = i0 + lane;
        float x = 0.0f;
        const bool ok = i < w_hi && take(i, x);
        const uint32_t key = rank_key(x);
        n_above += __popcll(__ballot(ok && (all || key > prefix)));
        n_equal += __popcll(__ballot(ok && !all && key == prefix));
    }
    if (lane == 0) s_cnt[wave][0] = n_above, s_cnt[wave][1] = n_equal;
    __syncthreads();
    int above_seen = 0, equal_seen = 0;
    for (int w = 0; w < wave; ++w) above_seen += s_cnt[w][0], equal_seen += s_cnt[w][1];
    for (int i0 = w_lo; i0 < w_hi; i0 += 64) {
        const int i = i0 + lane;
        float x = 0.0f;
        const bool ok = i < w_hi && take(i, x);
        const uint32_t key = rank_key(x);
        const bool above = ok && (all || key > prefix), equal = ok && !all && key == prefix;
        const unsigned long long above_mask = __ballot(above), equal_mask = __ballot(equal);
        const int rank = equal_seen + __popcll(equal_mask & below);      // the equals before this one
        if (above || (equal && rank < (int)want)) {
            const int place = above_seen + __popcll(above_mask & below) + min(rank, (int)want);
            if constexpr (LEVEL == 2) out[place] = pos[i];
            else out[place] = lo + i;
            if constexpr (LEVEL == 1) out_scores[place] = x;
        }
        above_seen += __popcll(above_mask), equal_seen += __popcll(equal_mask);
    }
    for (int i = min(valid, k) + tid; i < k; i += 256) out[i] = -1;
}


// The sum of s_wave[0 .. wave - 1] and of all 16 entries: lane l reads entry l % 16, a scan over the lanes, and the
// two sums are lanes wave - 1 and 15 of it (`wave` is uniform): a dozen instructions and one LDS round trip, where a
// loop over the entries before this wavefront's is up to fifteen round trips one after another.
PKV_DEV unsigned waves_before(const unsigned* s_wave, int wave, int lane, unsigned& total) {
    const unsigned v = s_wave[lane & 15];
    const unsigned incl = wave_inclusive_sum(v);
    total = (unsigned)__builtin_amdgcn_readlane((int)incl, 15);
    const unsigned upto = (unsigned)__builtin_amdgcn_readlane((int)incl, wave > 0 ? wave - 1 : 0);
    return wave > 0 ? upto : 0u;
}

template <int LEVEL, int EPT>
__global__ __launch_bounds__(1024) void index_topk_runs_kernel(TopkArgs a) {
    // Four copies of the histogram, a lane's by its number; a copy's bins side by side (a wavefront's lanes that fall into
    // different bins meet in different banks, and the scan reads a thread's bins as one word or two, no two lanes in a
    // bank), the copies 16 words out of step, so that a bin's four copies are four banks too.
    constexpr int COPIES = 4, COPY_WORDS = 2048 + 16;
    __shared__ __align__(16) unsigned s_hist[COPIES * COPY_WORDS];
    __shared__ __align__(16) unsigned s_wave[16];
    __shared__ unsigned s_pick[2];
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int t = blockIdx.x, part = LEVEL == 1 ? blockIdx.y : 0;
    const int end = min(max(a.ends[t], 0), a.n);
    const int k = a.k;
    const float* row = a.s + (int64_t)t * a.s_stride;
    const int32_t* pos = LEVEL == 2 ? a.pos + (int64_t)t * a.s_stride : nullptr;
    int32_t* out = a.out + (int64_t)t * a.out_stride + (int64_t)part * k;
    float* out_scores = LEVEL == 1 ? a.out_scores + (int64_t)t * a.out_stride + (int64_t)part * k : nullptr;
    int lo = 0, m, valid, avail;      // avail: the elements the row holds from lo on, whatever `end` says
    if constexpr (LEVEL == 2) {
        m = a.parts * k, valid = 0, avail = m;
        for (int p = 0; p < a.parts; ++p) valid += min(max(min(end - p * a.width, a.width), 0), k);
    } else {
        lo = LEVEL == 1 ? part * a.width : 0;
        m = max(min(LEVEL == 1 ? a.width : a.n, end - lo), 0), valid = m;
        avail = max(min(LEVEL == 1 ? a.width : a.n, a.n - lo), 0);
    }
    row += lo;
    const int first = tid * EPT;
    const bool mine = first < m;      // this thread's run holds elements of the row
    uint32_t key[EPT];
    int held_pos[LEVEL == 2 ? EPT : 1];      // LEVEL 2: the candidates' positions, kept for the writes
    using Bits = typename std::conditional<(EPT > 32), uint64_t, uint32_t>::type;
    Bits ok = 0;      // bit j: element first + j is a candidate
#pragma unroll
    for (int j = 0; j < EPT; ++j) key[j] = 0u;
    if (mine) {
        const bool whole = EPT % 4 == 0 && first + EPT <= avail && (reinterpret_cast<uintptr_t>(row) & 15) == 0 &&
                           (LEVEL != 2 || (reinterpret_cast<uintptr_t>(pos) & 15) == 0);
        constexpr int AT_ONCE = EPT > 32 ? EPT / 2 : EPT;      // (the loads in flight and the keys held share a thread's registers)
#pragma unroll
        for (int j0 = 0; j0 < EPT; j0 += AT_ONCE) {
            float x[AT_ONCE];
            int at[AT_ONCE];
            if (whole) {
                if constexpr (EPT % 4 == 0) {
#pragma unroll
                    for (int q = 0; q < AT_ONCE / 4; ++q) {
                        const f32x4 v = *reinterpret_cast<const f32x4*>(row + first + j0 + 4 * q);
                        x[4 * q] = v.x, x[4 * q + 1] = v.y, x[4 * q + 2] = v.z, x[4 * q + 3] = v.w;
                        if constexpr (LEVEL == 2) {
                            const u32x4 w = *reinterpret_cast<const u32x4*>(pos + first + j0 + 4 * q);
                            at[4 * q] = (int)w.x, at[4 * q + 1] = (int)w.y, at[4 * q + 2] = (int)w.z, at[4 * q + 3] = (int)w.w;
                        } else {
                            at[4 * q] = at[4 * q + 1] = at[4 * q + 2] = at[4 * q + 3] = 0;
                        }
                    }
                }
            } else {
#pragma unroll
                for (int jj = 0; jj < AT_ONCE; ++jj) {
                    const int i = first + j0 + jj;
                    x[jj] = i < m ? row[i] : 0.0f;
                    at[jj] = 0;
                    if constexpr (LEVEL == 2) at[jj] = i < m ? pos[i] : -1;
                }
            }
#pragma unroll
            for (int jj = 0; jj < AT_ONCE; ++jj) {
                const int j = j0 + jj;
                const bool is = first + j < m && at[jj] >= 0;
                key[j] = is ? rank_key(x[jj]) : 0u;
                if (is) ok |= (Bits)1 << j;
                if constexpr (LEVEL == 2) held_pos[j] = at[jj];
            }
        }
    }
    const bool all = valid <= k;      // everything is picked
    uint32_t prefix = 0u;
    unsigned want = 0u;               // of the keys equal to the k-th, the `want` first are taken
    if (!all) {
        want = (unsigned)k;
        static_for<3>([&](auto pass) {
            constexpr int p = pass;
            constexpr int kShift[3] = {21, 10, 0}, kDigit[3] = {11, 11, 10};
            constexpr int shift = kShift[p], bins = 1 << kDigit[p], done = shift + kDigit[p];      // `done`: the bits below the digits already chosen
            for (int i = tid; i < COPIES * COPY_WORDS / 4; i += 1024) reinterpret_cast<u32x4*>(s_hist)[i] = u32x4{0u, 0u, 0u, 0u};
            lds_barrier();
            if (mine) {
                unsigned* const copy = s_hist + (lane & (COPIES - 1)) * COPY_WORDS;
#pragma unroll
                for (int j = 0; j < EPT; ++j) {
                    if constexpr (p == 0) atomicAdd(&copy[key[j] >> 21], 1u);
                    else if ((key[j] >> (done & 31)) == (prefix >> (done & 31))) atomicAdd(&copy[(key[j] >> shift) & (unsigned)(bins - 1)], 1u);
                }
            }
            lds_barrier();
            // thread tid: the bins per * tid upwards (per of them); a scan of the counts from bin 0 up, and what lies
            // above a bin is the total less the scan up to it
            constexpr int per = bins / 1024;
            unsigned h[per], sum = 0u;
#pragma unroll
            for (int i = 0; i < per; ++i) h[i] = 0u;
#pragma unroll
            for (int c = 0; c < COPIES; ++c) {
                const unsigned* mine_of = s_hist + c * COPY_WORDS + per * tid;
                if constexpr (per % 4 == 0) {
#pragma unroll
                    for (int i = 0; i < per; i += 4) {
                        const u32x4 v = *reinterpret_cast<const u32x4*>(mine_of + i);
                        h[i] += v.x, h[i + 1] += v.y, h[i + 2] += v.z, h[i + 3] += v.w;
                    }
                } else if constexpr (per == 2) {
                    const u32x2 v = *reinterpret_cast<const u32x2*>(mine_of);
                    h[0] += v.x, h[1] += v.y;
                } else {
                    h[0] += mine_of[0];
                }
            }
#pragma unroll
            for (int i = 0; i < per; ++i) sum += h[i];
            unsigned incl = wave_inclusive_sum(sum);
            if (lane == 63) s_wave[wave] = incl;
            lds_barrier();
            unsigned total;
            incl += waves_before(s_wave, wave, lane, total);
            unsigned before = total - incl;      // the keys in the bins above this thread's
#pragma unroll
            for (int i = per - 1; i >= 0; --i) {
                const unsigned upto = before + h[i];
                if (upto >= want && before < want) s_pick[0] = (unsigned)(tid * per + i), s_pick[1] = want - before;
                before = upto;
            }
            lds_barrier();
            prefix |= s_pick[0] << shift;
            want = s_pick[1];
        });
    }
    // What each thread writes (above the k-th key | equal to it << 16), then the places before each thread's. A key of
    // 0 is a NaN's or that of an element that is no candidate: only where the k-th key is 0 (or everything is picked)
    // does an element's bit of `ok` decide.
    const bool plain = !all && prefix != 0u;
    auto is_above = [&](int j) __attribute__((always_inline)) -> bool {
        return plain ? key[j] > prefix : (((ok >> j) & 1u) && (all || key[j] > prefix));
    };
    auto is_equal = [&](int j) __attribute__((always_inline)) -> bool {
        return plain ? key[j] == prefix : (((ok >> j) & 1u) && !all && key[j] == prefix);
    };
    unsigned n_above = 0u, n_equal = 0u;
    if (plain) {
#pragma unroll
        for (int j = 0; j < EPT; ++j) n_above += key[j] > prefix ? 1u : 0u, n_equal += key[j] == prefix ? 1u : 0u;
    } else {
#pragma unroll
        for (int j = 0; j < EPT; ++j) n_above += is_above(j) ? 1u : 0u, n_equal += is_equal(j) ? 1u : 0u;
    }
    const unsigned both = n_above | (n_equal << 16);      // (a row holds fewer than 65,536 elements: no carry between the halves)
    unsigned incl = wave_inclusive_sum(both);
    if (lane == 63) s_wave[wave] = incl;
    lds_barrier();
    unsigned total;
    incl += waves_before(s_wave, wave, lane, total);
    int above_seen = (int)((incl - both) & 0xffffu), equal_seen = (int)((incl - both) >> 16);
    const int picks = min(valid, k);
    if (n_above | n_equal) {
        int place = above_seen + min(equal_seen, (int)want);      // (one further for every element written)
#pragma unroll
        for (int j = 0; j < EPT; ++j) {
            const bool above = is_above(j), equal = is_equal(j);
            if (above || (equal && equal_seen < (int)want)) {
                out[place] = LEVEL == 2 ? held_pos[j] : lo + first + j;
                if constexpr (LEVEL == 1) out_scores[place] = score_of_key(key[j]);
                ++place;
            }
            equal_seen += equal ? 1 : 0;
        }
    }
    for (int i = picks + tid; i < k; i += 1024) out[i] = -1;
}

template <bool F16, bool FP8, int HT, int KS>
int launch_scores_shape(ScoreArgs a, bool many, int cus, hipStream_t stream) {
    if (!many) {
        // A block of keys a workgroup, sized so that the workgroups are as many as the chip holds at once (or a whole
        // number of times that many): every one runs from the start and they end together. Three tiles in flight a
        // wavefront where the queries leave the registers room and a wavefront has 64 tiles or more (measured: 64
        // sequences of 50,000 keys in place 201 us against 207 with one tile in flight, E4M3 rows 124 against 139;
        // blocks shorter than that are faster with one and a third workgroup a compute unit, 16 sequences 43 us
        // against 45, 4 tokens 13.9 against 14.9).
        static int held_at_once[2] = {0, 0};      // workgroups a compute unit holds, by kernel (the chips of a process are alike)
        auto resident = [&](int deep) -> int {
            if (!held_at_once[deep]) {
                int count = 0;
                const hipError_t e = deep ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&count, index_scores_kernel<F16, FP8, HT, KS, 3>, 256, 0)
                                          : hipOccupancyMaxActiveBlocksPerMultiprocessor(&count, index_scores_kernel<F16, FP8, HT, KS, 1>, 256, 0);
                held_at_once[deep] = e == hipSuccess && count > 0 ? count : 1;
            }
            return held_at_once[deep];
        };
        auto block_for = [&](int deep) -> int {
            const int64_t room = (int64_t)cus * resident(deep);
            const int64_t fewest = ((int64_t)a.n + 8191) / 8192;      // blocks a token: none above 8,192 keys
            const int64_t rounds = max((fewest * a.tokens + room - 1) / room, (int64_t)1);
            const int64_t blocks = max(room * rounds / a.tokens, fewest);
            return (int)(((a.n + blocks - 1) / blocks + 63) / 64 * 64);
        };
        const bool room_for_three = HT * KS <= 32;
        int block = block_for(room_for_three ? 1 : 0);
        const bool deep = room_for_three && block >= 4096;
        if (room_for_three && !deep) block = block_for(0);
        a.block = block;
        const dim3 grid((unsigned)((a.n + block - 1) / block), (unsigned)a.tokens);
        if (deep) hipLaunchKernelGGL((index_scores_kernel<F16, FP8, HT, KS, 3>), grid, dim3(256), 0, stream, a);
        else hipLaunchKernelGGL((index_scores_kernel<F16, FP8, HT, KS, 1>), grid, dim3(256), 0, stream, a);
        return hip_code(hipGetLastError());
    }
    constexpr int TW = HT * KS <= 16 && HT <= 4 ? 2 : 1;      // two tokens a wavefront where their queries fit its registers
    constexpr int E = FP8 ? 1 : 2;
    constexpr size_t lds = (size_t)4 * TW * HT * 16 * 4 + 2 * 64 * (KS * 32 * E + 16);
    const int wgs_t = (a.tokens + 4 * TW - 1) / (4 * TW);
    int block = 256;
    while (block < 8192 && (int64_t)wgs_t * ((a.n + block - 1) / block) > (int64_t)cus * 16) block *= 2;
    a.block = block;
    if (lds > 48 * 1024) {
        static bool raised[16] = {};      // per device: the kernel's LDS limit
        int device = 0;
        if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 16) return CRIT_PKV_E_GEOMETRY;
        if (!raised[device]) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(&index_scores_tokens_kernel<F16, FP8, HT, KS, TW>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
                return CRIT_PKV_E_GEOMETRY;
            raised[device] = true;
        }
    }
    const dim3 grid((unsigned)((a.n + block - 1) / block), (unsigned)wgs_t);
    hipLaunchKernelGGL((index_scores_tokens_kernel<F16, FP8, HT, KS, TW>), grid, dim3(256), lds, stream, a);
    return hip_code(hipGetLastError());
}

template <bool F16, bool FP8>
int launch_scores_kind(const ScoreArgs& a, int dim, bool many, int cus, hipStream_t stream) {
    const int ht = (a.heads + 15) / 16;
#define PKV_SHAPE(H, K) if (ht == H && dim == K * 32) return launch_scores_shape<F16, FP8, H, K>(a, many, cus, stream);
    PKV_SHAPE(1, 2) PKV_SHAPE(1, 4) PKV_SHAPE(1, 8)
    PKV_SHAPE(2, 2) PKV_SHAPE(2, 4) PKV_SHAPE(2, 8)
    PKV_SHAPE(4, 2) PKV_SHAPE(4, 4) PKV_SHAPE(4, 8)
    PKV_SHAPE(8, 2) PKV_SHAPE(8, 4) PKV_SHAPE(8, 8)
#undef PKV_SHAPE
    return CRIT_PKV_E_GEOMETRY;
}

// How a call selects. held: the elements a workgroup holds in registers (1,024 threads x 8, 16 or 32). A row that fits
// is one workgroup's; a longer row goes in slices of `width` positions (each a workgroup's), then the slices' picks
// (parts x k candidates, which must fit a workgroup too), where the candidates' room stays within kSliceRoom; everything
// else streams, a workgroup a row.
constexpr int kHeld = 32768;
// Calls of many rows hold rows of up to kHeldWide elements whole, a workgroup a row (no slices, no candidates' pass:
// measured for rows of 50,000 and k = 2,048: 253 against 432 us in slices for 2,048 rows, 37 against 58 for 256; 64 rows
// take 22 us in slices, which spread a row over compute units, and 38 whole). Short of 65,536 so that the counts of
// the keys above and equal to the k-th fit 16 bits each.
constexpr int kHeldWide = 64512;
constexpr int kManyRows = 128;
constexpr int64_t kSliceRoom = (int64_t)512 << 20;
struct TopkPlan {
    int parts;      // 0: one pass a row
    int width;
};
// Elements a thread of the holding kernel for `elements` of a row (what launch_topk_level picks).
int held_elements(int elements) {
    const int steps[] = {8, 12, 16, 24, 32};
    for (int e : steps)
        if (elements <= e * 1024) return e;
    return 0;
}
TopkPlan topk_plan(int tokens, int n, int k, int cus) {
    TopkPlan plan = {0, n};
    (void)cus;
    if (n <= kHeld || tokens > 65535 || (n <= kHeldWide && tokens >= kManyRows)) return plan;
    // Slices: the fewest microseconds by what the holding kernel was measured to take, 4.3 us and 0.42 us an element
    // a thread (the candidates' pass, which also loads positions, 1.15 times that): for a few rows the two launches one
    // after the other, for many rows every slice's workgroup counts. (50,000 positions, k = 2,048: 4 slices of 12,544
    // and 8,192 candidates, 20 us.)
    const int64_t fewest = ((int64_t)n + kHeld - 1) / kHeld;
    const int64_t most = min((int64_t)kHeld / k, min((int64_t)65535, max(fewest * 8, (int64_t)16)));
    float best = 0.0f;
    for (int64_t parts = max(fewest, (int64_t)2); parts <= most; ++parts) {
        const int width = (int)((((int64_t)n + parts - 1) / parts + 63) / 64 * 64);
        const int e1 = held_elements(width), e2 = held_elements((int)(parts * k));
        if (!e1 || !e2 || (int64_t)tokens * parts * k * 8 > kSliceRoom) continue;
        const float slices = 4.3f + 0.42f * e1, candidates = 1.15f * (4.3f + 0.42f * e2);
        const float cost = (tokens >= kManyRows ? (float)parts : 1.0f) * slices + candidates;
        if (plan.parts == 0 || cost < best) best = cost, plan.parts = (int)parts, plan.width = width;
    }
    return plan;
}

template <int LEVEL>
void launch_topk_level(const TopkArgs& a, int elements, dim3 grid, hipStream_t stream) {
    // (elements a thread: threads past the row's end skip the passes, so the count only has to hold the row)
#define PKV_RUNS(L, E) hipLaunchKernelGGL((index_topk_runs_kernel<L, E>), grid, dim3(1024), 0, stream, a)
    if (elements <= 8192) PKV_RUNS(LEVEL, 8);
    else if (elements <= 12288) PKV_RUNS(LEVEL, 12);
    else if (elements <= 16384) PKV_RUNS(LEVEL, 16);
    else if (elements <= 24576) PKV_RUNS(LEVEL, 24);
    else if (elements <= kHeld) PKV_RUNS(LEVEL, 32);
    else if (LEVEL == 0 && elements <= 40960 && (int)grid.x >= kManyRows) PKV_RUNS(0, 40);
    else if (LEVEL == 0 && elements <= 49152 && (int)grid.x >= kManyRows) PKV_RUNS(0, 48);
    else if (LEVEL == 0 && elements <= 57344 && (int)grid.x >= kManyRows) PKV_RUNS(0, 56);
    else if (LEVEL == 0 && elements <= kHeldWide && (int)grid.x >= kManyRows) PKV_RUNS(0, 64);
    else hipLaunchKernelGGL(index_topk_kernel<LEVEL>, grid, dim3(256), 0, stream, a);
#undef PKV_RUNS
}

}   // namespace

int launch_index_scores(const crit_pkv_index_scores_params* p, hipStream_t stream) {
    if (!p || !p->q || !p->keys || !p->weights || !p->ends || !p->out) return CRIT_PKV_E_NULL;
    if (p->tokens == 0 || p->n == 0) return 0;
    const bool fp8 = p->key_dtype == 2;
    if (p->key_dtype < 0 || p->key_dtype > 2 || (p->q_dtype != CRIT_PKV_BF16 && p->q_dtype != CRIT_PKV_F16)) return CRIT_PKV_E_DTYPE;
    if (!fp8 && p->key_dtype != (p->q_dtype == CRIT_PKV_F16 ? 1 : 0)) return CRIT_PKV_E_DTYPE;
    if (fp8 && !p->key_scales) return CRIT_PKV_E_NULL;
    if (p->tokens < 0 || p->tokens > 65535 || p->n < 0 || p->n > (1 << 30) || p->heads < 1 || p->heads > 128 ||
        (p->dim != 64 && p->dim != 128 && p->dim != 256) || p->group < 1 || p->q_stride_t % 8 || p->q_stride_h % 8 ||
        (reinterpret_cast<uintptr_t>(p->q) % 16) || (reinterpret_cast<uintptr_t>(p->keys) % 16) || p->key_stride % (fp8 ? 16 : 8) ||
        p->out_stride < p->n)
        return CRIT_PKV_E_GEOMETRY;
    ScoreArgs a;
    a.q = reinterpret_cast<const uint8_t*>(p->q), a.keys = reinterpret_cast<const uint8_t*>(p->keys);
    a.key_scales = p->key_scales, a.weights = p->weights, a.ends = p->ends, a.slots = p->slots, a.out = p->out;
    a.q_st = p->q_stride_t, a.q_sh = p->q_stride_h, a.key_stride = p->key_stride, a.w_stride = p->weights_stride;
    a.out_stride = p->out_stride, a.slots_stride = p->slots_stride;
    a.tokens = p->tokens, a.n = p->n, a.group = p->group, a.heads = p->heads, a.slots_are_64 = p->slots_are_64;
    a.scale = p->scale, a.block = 64;
    const int cus = compute_units() > 0 ? compute_units() : 256;
    // many tokens share their keys through LDS, 4 or 8 to a workgroup: where the keys are read in place, a group's
    // tokens (they share the slots) must fill workgroups, unless one list serves every token (slots_stride 0)
    const int ht = (p->heads + 15) / 16;
    const int wg_tokens = ht * (p->dim / 32) <= 16 && ht <= 4 ? 8 : 4;
    const bool many = p->tokens >= 16 && (!p->slots || p->slots_stride == 0 || p->group % wg_tokens == 0);
    const bool f16 = p->q_dtype == CRIT_PKV_F16;
    if (fp8) return f16 ? launch_scores_kind<true, true>(a, p->dim, many, cus, stream) : launch_scores_kind<false, true>(a, p->dim, many, cus, stream);
    return f16 ? launch_scores_kind<true, false>(a, p->dim, many, cus, stream) : launch_scores_kind<false, false>(a, p->dim, many, cus, stream);
}

int64_t index_topk_work_bytes(int tokens, int n, int k) {
    if (tokens <= 0 || n <= 0 || k <= 0) return 0;
    const TopkPlan plan = topk_plan(tokens, n, k, compute_units() > 0 ? compute_units() : 256);
    return (int64_t)tokens * plan.parts * k * 8;
}

int launch_index_topk(const crit_pkv_index_topk_params* p, hipStream_t stream) {
    if (!p || !p->scores || !p->ends || !p->out) return CRIT_PKV_E_NULL;
    if (p->tokens == 0) return 0;
    if (p->tokens < 0 || p->n < 0 || p->n > (1 << 30) || p->k < 1 || p->scores_stride < p->n || p->out_stride < p->k) return CRIT_PKV_E_GEOMETRY;
    TopkArgs a;
    a.s = p->scores, a.pos = nullptr, a.ends = p->ends, a.out = p->out, a.out_scores = nullptr;
    a.s_stride = p->scores_stride, a.out_stride = p->out_stride;
    a.tokens = p->tokens, a.n = p->n, a.k = p->k, a.width = p->n, a.parts = 1;
    const TopkPlan plan = topk_plan(p->tokens, p->n, p->k, compute_units() > 0 ? compute_units() : 256);
    const int64_t need = (int64_t)p->tokens * plan.parts * p->k * 8;
    if (plan.parts > 1 && p->work && p->work_bytes >= need) {
        // the slices' k best (positions, then scores: [tokens][parts][k] each), then the k best of those
        int32_t* cand = reinterpret_cast<int32_t*>(p->work);
        float* cand_scores = reinterpret_cast<float*>(cand + (int64_t)p->tokens * plan.parts * p->k);
        TopkArgs s1 = a;
        s1.out = cand, s1.out_scores = cand_scores, s1.out_stride = (int64_t)plan.parts * p->k, s1.width = plan.width, s1.parts = plan.parts;
        launch_topk_level<1>(s1, plan.width, dim3((unsigned)p->tokens, (unsigned)plan.parts), stream);
        TopkArgs s2 = a;
        s2.s = cand_scores, s2.pos = cand, s2.s_stride = (int64_t)plan.parts * p->k, s2.width = plan.width, s2.parts = plan.parts;
        launch_topk_level<2>(s2, plan.parts * p->k, dim3((unsigned)p->tokens), stream);
        return hip_code(hipGetLastError());
    }
    launch_topk_level<0>(a, p->n, dim3((unsigned)p->tokens), stream);
    return hip_code(hipGetLastError());
}

}   // namespace pkv
