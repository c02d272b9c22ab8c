// Append to a latent cache: each token's latent (rank values) and rotary key (rope values) stored side by side in the
// token's slot of cache [slots][rank + rope], in the cache's type. What the reference's latent-attention module does
// with torch indexing (kernels/techniques/attention/latent-attention/torch-ext/latent_attention/__init__.py:74-97):
// 16-bit caches take the values rounded to nearest even; an E4M3 cache codes each of the two parts at its own scale,
// scale = max(amax / 448, 1e-30) and code = e4m3(clamp(x / scale, -448, 448)), both divisions IEEE, and keeps the two
// scales in scales [slots][2]. One launch; one wavefront a token, its lanes striding over the row, so reads and writes
// are contiguous. HBM-bound, and small: a decode step appends one row a sequence.
#include "pkv_common.hpp"
#include "pkv_launch.hpp"

namespace pkv {
namespace {

struct LatentWriteArgs {
    const void* part[2];      // the latent, the rotary key
    int64_t stride[2];        // elements between two tokens' rows
    int width[2];
    const int64_t* slots;
    uint8_t* cache;
    float* scales;
    int64_t tokens;
};

template <int IN>
PKV_DEV float in_value(const void* base, int64_t i) {
    if constexpr (IN == CRIT_PKV_F32) return reinterpret_cast<const float*>(base)[i];
    if constexpr (IN == CRIT_PKV_BF16) return u2f((uint32_t)reinterpret_cast<const uint16_t*>(base)[i] << 16);
    return (float)reinterpret_cast<const _Float16*>(base)[i];
}

// The larger of two magnitudes, a NaN winning over every number (torch's amax).
PKV_DEV float nan_max(float a, float b) { return (b > a || b != b) ? b : a; }

// CACHE: 0 BF16, 1 FP16, 2 E4M3.
template <int IN, int CACHE>
__global__ __launch_bounds__(256) void latent_write_kernel(LatentWriteArgs a) {
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (t >= a.tokens) return;
    const int64_t slot = a.slots[t];
    if (slot < 0) return;      // (a token with no slot is skipped, as the KV append skips it)
    const int row_width = a.width[0] + a.width[1];
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const void* src = a.part[which];
        const int64_t from = t * a.stride[which];
        const int n = a.width[which];
        const int64_t to = slot * row_width + (which ? a.width[0] : 0);
        if constexpr (CACHE < 2) {
            uint16_t* dst = reinterpret_cast<uint16_t*>(a.cache) + to;
            if constexpr ((IN == CRIT_PKV_BF16 && CACHE == 0) || (IN == CRIT_PKV_F16 && CACHE == 1)) {
                // rows of the cache's own type are stored as they are, every bit (the reference's .to() of the same
                // dtype is the tensor itself: a NaN keeps its payload)
                for (int i = lane; i < n; i += 64) dst[i] = reinterpret_cast<const uint16_t*>(src)[from + i];
            } else {
                for (int i = lane; i < n; i += 64) {
                    const float x = in_value<IN>(src, from + i);
                    dst[i] = (uint16_t)(CACHE == 1 ? f16_bits(x) : bf16_rne(x));
                }
            }
        } else {
            float amax = 0.0f;
            for (int i = lane; i < n; i += 64) amax = nan_max(amax, __builtin_fabsf(in_value<IN>(src, from + i)));
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) amax = nan_max(amax, __shfl_xor(amax, o));
            float scale = __fdiv_rn(amax, 448.0f);
            scale = scale < 1e-30f ? 1e-30f : scale;      // (a NaN stays)
            if (lane == 0) a.scales[slot * 2 + which] = scale;
            uint8_t* dst = a.cache + to;
            for (int i = lane; i < n; i += 64) dst[i] = (uint8_t)e4m3_encode(__fdiv_rn(in_value<IN>(src, from + i), scale));
        }
    }
}

template <int IN>
int launch_in(const LatentWriteArgs& a, int cache_dtype, hipStream_t stream) {
    const dim3 grid((unsigned)((a.tokens + 3) / 4));
    switch (cache_dtype) {
        case 0: hipLaunchKernelGGL((latent_write_kernel<IN, 0>), grid, dim3(256), 0, stream, a); break;
        case 1: hipLaunchKernelGGL((latent_write_kernel<IN, 1>), grid, dim3(256), 0, stream, a); break;
        case 2: hipLaunchKernelGGL((latent_write_kernel<IN, 2>), grid, dim3(256), 0, stream, a); break;
        default: return CRIT_PKV_E_DTYPE;
    }
    return hip_code(hipGetLastError());
}

}   // namespace

int launch_latent_write(const crit_pkv_latent_write_params* p, hipStream_t stream) {
    if (!p || !p->latent || !p->rope || !p->slots || !p->cache) return CRIT_PKV_E_NULL;
    if (p->cache_dtype == 2 && !p->scales) return CRIT_PKV_E_NULL;
    if (p->tokens < 0 || p->rank < 1 || p->rope_width < 1 || p->latent_stride < p->rank || p->rope_stride < p->rope_width ||
        (p->tokens + 3) / 4 > 0x7fffffff)
        return CRIT_PKV_E_GEOMETRY;
    if (p->tokens == 0) return 0;
    LatentWriteArgs a;
    a.part[0] = p->latent, a.part[1] = p->rope;
    a.stride[0] = p->latent_stride, a.stride[1] = p->rope_stride;
    a.width[0] = p->rank, a.width[1] = p->rope_width;
    a.slots = p->slots, a.cache = reinterpret_cast<uint8_t*>(p->cache), a.scales = p->scales, a.tokens = p->tokens;
    switch (p->in_dtype) {
        case CRIT_PKV_F32: return launch_in<CRIT_PKV_F32>(a, p->cache_dtype, stream);
        case CRIT_PKV_BF16: return launch_in<CRIT_PKV_BF16>(a, p->cache_dtype, stream);
        case CRIT_PKV_F16: return launch_in<CRIT_PKV_F16>(a, p->cache_dtype, stream);
    }
    return CRIT_PKV_E_DTYPE;
}

}   // namespace pkv
