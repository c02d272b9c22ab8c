// Sparse index selection for gfx950: every query token's score over the compressed keys it may see, and the positions
// of its k best, which a block-sparse attention then reads. What the reference's sparse-indexer kernels module computes
// (kernels/techniques/attention/sparse-indexer/torch-ext/sparse_indexer/__init__.py:83-139, _kernels.py; the operation:
// inference/attention-state/code/sparse_index.py):
//   score[t][s] = sum_h weights[t][h] * scale * max(0, q[t][h] . keys[s])   for s < ends[t], -inf at or past it
//   picked[t]   = the positions of the k largest scores below ends[t], ascending, then -1; ties to the lower position,
//                 a NaN below every number
//
// index_scores_kernel: a workgroup is one token and a block of keys; each of its four wavefronts takes tiles of 16 keys.
// The token's queries sit in LDS (heads x dim, 16-bit); a tile's key rows are loaded as they lie (a lane: one key, 8
// adjacent values per k-step: the A operand of v_mfma_f32_16x16x32), from their slots where the keys are read in place.
// S^T = K Q^T per tile of 16 heads leaves a lane one head's products with 4 keys: ReLU, the head's factor, then the sum
// over the 16 heads as a fixed tree of lane exchanges, the head tiles added in order. So a token's bits are its own:
// not its neighbours', not the launch's shape.
//
// index_topk_kernel: a workgroup a token. The scores map to 32-bit keys that order as the rule does (NaN lowest, -0 = +0),
// an 8-bit radix select from the top finds the k-th key and how many of its equals are taken, and one pass in position
// order writes the positions of everything above it and of its first equals: ascending by construction.
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
    int tokens, n, group, heads, dim, slots_are_64, block;
    float scale;
};

template <bool F16, bool FP8>
__global__ __launch_bounds__(256) void index_scores_kernel(ScoreArgs a) {
    extern __shared__ __align__(16) uint8_t s_q[];      // [heads padded to 16][dim * 2 + 32 bytes]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, g = lane >> 4, li = lane & 15;
    const int t = blockIdx.y;
    const int d = a.dim, H = a.heads;
    const int rowb = d * 2 + 32;
    const int hp = (H + 15) / 16 * 16;
    // the token's queries, heads past the last as zeros
    const int chunks = d / 8;
    for (int i = tid; i < hp * chunks; i += 256) {
        const int h = i / chunks, c = i - h * chunks;
        u32x4 w = {0u, 0u, 0u, 0u};
        if (h < H) w = *reinterpret_cast<const u32x4*>(a.q + ((int64_t)t * a.q_st + (int64_t)h * a.q_sh) * 2 + c * 16);
        *reinterpret_cast<u32x4*>(s_q + h * rowb + c * 16) = w;
    }
    __syncthreads();
    const int end = min(max(a.ends[t], 0), a.n);
    const int ksteps = d / 32;
    const int64_t srow = (int64_t)(t / a.group) * a.slots_stride;
    const int first = blockIdx.x * a.block;
    const int last = min(first + a.block, a.n);
    for (int k0 = first + wave * 16; k0 < last; k0 += 64) {
        float* out = a.out + (int64_t)t * a.out_stride;
        if (k0 >= end) {      // nothing of the tile is seen
            if (g == 0 && k0 + li < last) out[k0 + li] = -INFINITY;
            continue;
        }
        // the lane's key (the tile's row li), a key past the last reads the last
        const int key = min(k0 + li, a.n - 1);
        int64_t at = key;
        if (a.slots) at = a.slots_are_64 ? reinterpret_cast<const int64_t*>(a.slots)[srow + key] : (int64_t) reinterpret_cast<const int32_t*>(a.slots)[srow + key];
        const uint8_t* krow = a.keys + at * a.key_stride * (FP8 ? 1 : 2) + g * (FP8 ? 8 : 16);
        u32x4 ka[8];      // up to 8 k-steps (dim 256)
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            if (ks < ksteps) {
                if constexpr (FP8) {
                    const u32x2 c = *reinterpret_cast<const u32x2*>(krow + ks * 32);
                    const f32x2 a0 = e4m3_pair<false>(c.x), a1 = e4m3_pair<true>(c.x), a2 = e4m3_pair<false>(c.y), a3 = e4m3_pair<true>(c.y);
                    ka[ks] = u32x4{pair16<F16>(a0.x, a0.y), pair16<F16>(a1.x, a1.y), pair16<F16>(a2.x, a2.y), pair16<F16>(a3.x, a3.y)};
                } else {
                    ka[ks] = *reinterpret_cast<const u32x4*>(krow + ks * 64);
                }
            }
        }
        float total[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int ht = 0; ht < hp / 16; ++ht) {
            f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
            const uint8_t* qrow = s_q + (ht * 16 + li) * rowb + g * 16;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks)
                if (ks < ksteps) acc = mfma_k32<F16>(ka[ks], *reinterpret_cast<const u32x4*>(qrow + ks * 64), acc);
            const int h = ht * 16 + li;
            const float factor = h < H ? a.weights[(int64_t)t * a.w_stride + h] * a.scale : 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float v = __builtin_fmaxf(acc[i], 0.0f) * factor;
                // the 16 heads of the tile: a tree over the lanes 1, 2, 4, 8 apart
                v += __shfl_xor(v, 1);
                v += __shfl_xor(v, 2);
                v += __shfl_xor(v, 4);
                v += __shfl_xor(v, 8);
                total[i] += v;
            }
        }
        if (li < 4) {      // lane li of quarter g writes key 4 g + li
            const int kk = k0 + 4 * g + li;
            float v = li == 0 ? total[0] : (li == 1 ? total[1] : (li == 2 ? total[2] : total[3]));
            if constexpr (FP8) {
                const int key2 = min(kk, a.n - 1);
                int64_t at2 = key2;
                if (a.slots) at2 = a.slots_are_64 ? reinterpret_cast<const int64_t*>(a.slots)[srow + key2] : (int64_t) reinterpret_cast<const int32_t*>(a.slots)[srow + key2];
                v *= a.key_scales[at2];
            }
            if (kk < last) out[kk] = kk < end ? v : -INFINITY;
        }
    }
}

struct TopkArgs {
    const float* s;
    const int32_t* ends;
    int32_t* out;
    int64_t s_stride, out_stride;
    int tokens, n, k;
};

// The key a score is ranked by: larger first; -0 and +0 the same; -inf below every finite; a NaN below everything.
PKV_DEV uint32_t rank_key(float x) {
    if (x != x) return 0u;
    uint32_t u = f2u(x == 0.0f ? 0.0f : x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__global__ __launch_bounds__(256) void index_topk_kernel(TopkArgs a) {
    __shared__ unsigned s_hist[256];
    __shared__ unsigned s_pick[2];
    __shared__ int s_scan[2][4];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int t = blockIdx.x;
    const float* row = a.s + (int64_t)t * a.s_stride;
    int32_t* out = a.out + (int64_t)t * a.out_stride;
    const int end = min(max(a.ends[t], 0), a.n);
    const int k = a.k;
    if (end <= k) {
        for (int i = tid; i < k; i += 256) out[i] = i < end ? i : -1;
        return;
    }
    // radix select: the k-th largest key, 8 bits at a time from the top
    uint32_t prefix = 0u, mask = 0u;
    unsigned want = (unsigned)k;      // of the keys that match the prefix, the `want` largest are taken
    for (int shift = 24; shift >= 0; shift -= 8) {
        s_hist[tid] = 0u;
        __syncthreads();
        for (int i = tid; i < end; i += 256) {
            const uint32_t key = rank_key(row[i]);
            if ((key & mask) == prefix) atomicAdd(&s_hist[(key >> shift) & 255u], 1u);
        }
        __syncthreads();
        if (tid == 0) {
            unsigned above = 0u;
            int b = 255;
            for (; b > 0; --b) {
                if (above + s_hist[b] >= want) break;
                above += s_hist[b];
            }
            s_pick[0] = (unsigned)b, s_pick[1] = want - above;
        }
        __syncthreads();
        prefix |= s_pick[0] << shift;
        mask |= 255u << shift;
        want = s_pick[1];
        __syncthreads();
    }
    // positions in order: everything above the k-th key, and its first `want` equals
    int taken = 0, equals = 0;      // before this pass of 256 positions
    for (int i0 = 0; i0 < end; i0 += 256) {
        const int i = i0 + tid;
        const uint32_t key = i < end ? rank_key(row[i]) : 0u;
        const bool above = i < end && key > prefix, equal = i < end && key == prefix;
        const unsigned long long eq_mask = __ballot(equal), ab_mask = __ballot(above);
        const unsigned long long below = (1ull << lane) - 1ull;
        if (lane == 0) s_scan[0][wave] = __popcll(eq_mask), s_scan[1][wave] = __popcll(ab_mask);
        __syncthreads();
        int eq_before = equals, eq_total = equals;
        for (int w = 0; w < 4; ++w) {
            if (w < wave) eq_before += s_scan[0][w];
            eq_total += s_scan[0][w];
        }
        const int eq_rank = eq_before + __popcll(eq_mask & below);
        const bool pick = above || (equal && eq_rank < (int)want);
        // the picked ones of this pass, in order: the above, and the equals still wanted
        const int eq_picked_before_wave = min(eq_before, (int)want) - min(equals, (int)want);
        int ab_before = 0, ab_total = 0;
        for (int w = 0; w < 4; ++w) {
            if (w < wave) ab_before += s_scan[1][w];
            ab_total += s_scan[1][w];
        }
        const int eq_in_wave = min(eq_rank, (int)want) - min(eq_before, (int)want);
        const int place = taken + ab_before + eq_picked_before_wave + __popcll(ab_mask & below) + eq_in_wave;
        if (pick) out[place] = i;
        taken += ab_total + (min(eq_total, (int)want) - min(equals, (int)want));
        equals = eq_total;
        __syncthreads();
    }
}

}   // namespace

int launch_index_scores(const crit_pkv_index_scores_params* p, hipStream_t stream) {
    if (!p || !p->q || !p->keys || !p->weights || !p->ends || !p->out) return CRIT_PKV_E_NULL;
    if (p->tokens == 0 || p->n == 0) return 0;
    const bool fp8 = p->key_dtype == 2;
    if (p->key_dtype < 0 || p->key_dtype > 2 || (p->q_dtype != CRIT_PKV_BF16 && p->q_dtype != CRIT_PKV_F16)) return CRIT_PKV_E_DTYPE;
    if (!fp8 && p->key_dtype != (p->q_dtype == CRIT_PKV_F16 ? 1 : 0)) return CRIT_PKV_E_DTYPE;
    if (fp8 && !p->key_scales) return CRIT_PKV_E_NULL;
    if (p->tokens < 0 || p->tokens > 65535 || p->n < 0 || p->heads < 1 || p->heads > 128 || (p->dim != 64 && p->dim != 128 && p->dim != 256) ||
        p->group < 1 || p->q_stride_t % 8 || p->q_stride_h % 8 || (reinterpret_cast<uintptr_t>(p->q) % 16) ||
        (reinterpret_cast<uintptr_t>(p->keys) % 16) || p->key_stride % (fp8 ? 16 : 8) || p->out_stride < p->n)
        return CRIT_PKV_E_GEOMETRY;
    ScoreArgs a;
    a.q = reinterpret_cast<const uint8_t*>(p->q), a.keys = reinterpret_cast<const uint8_t*>(p->keys);
    a.key_scales = p->key_scales, a.weights = p->weights, a.ends = p->ends, a.slots = p->slots, a.out = p->out;
    a.q_st = p->q_stride_t, a.q_sh = p->q_stride_h, a.key_stride = p->key_stride, a.w_stride = p->weights_stride;
    a.out_stride = p->out_stride, a.slots_stride = p->slots_stride;
    a.tokens = p->tokens, a.n = p->n, a.group = p->group, a.heads = p->heads, a.dim = p->dim, a.slots_are_64 = p->slots_are_64;
    a.scale = p->scale;
    // a block of keys a workgroup: enough workgroups for the chip where the tokens are few, long blocks where they are many
    const int cus = compute_units();
    int block = 64;
    while (block < 4096 && (int64_t)p->tokens * ((p->n + block - 1) / block) > (int64_t)(cus > 0 ? cus : 256) * 16) block *= 2;
    a.block = block;
    const int hp = (p->heads + 15) / 16 * 16;
    const size_t lds = (size_t)hp * (p->dim * 2 + 32);
    const dim3 grid((unsigned)((p->n + block - 1) / block), (unsigned)p->tokens);
    const bool f16 = p->q_dtype == CRIT_PKV_F16;
#define PKV_SCORES(F, E)                                                                                              \
    {                                                                                                                  \
        if (lds > 48 * 1024)                                                                                           \
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(&index_scores_kernel<F, E>),                         \
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)               \
                return CRIT_PKV_E_GEOMETRY;                                                                            \
        hipLaunchKernelGGL((index_scores_kernel<F, E>), grid, dim3(256), lds, stream, a);                              \
    }
    if (fp8) {
        if (f16) PKV_SCORES(true, true) else PKV_SCORES(false, true)
    } else {
        if (f16) PKV_SCORES(true, false) else PKV_SCORES(false, false)
    }
#undef PKV_SCORES
    return hip_code(hipGetLastError());
}

int launch_index_topk(const crit_pkv_index_topk_params* p, hipStream_t stream) {
    if (!p || !p->scores || !p->ends || !p->out) return CRIT_PKV_E_NULL;
    if (p->tokens == 0) return 0;
    if (p->tokens < 0 || p->n < 0 || p->k < 1 || p->scores_stride < p->n || p->out_stride < p->k) return CRIT_PKV_E_GEOMETRY;
    TopkArgs a;
    a.s = p->scores, a.ends = p->ends, a.out = p->out, a.s_stride = p->scores_stride, a.out_stride = p->out_stride;
    a.tokens = p->tokens, a.n = p->n, a.k = p->k;
    hipLaunchKernelGGL(index_topk_kernel, dim3((unsigned)p->tokens), dim3(256), 0, stream, a);
    return hip_code(hipGetLastError());
}

}   // namespace pkv
