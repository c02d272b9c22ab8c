// KV append: a step's keys and values scattered into their slots of one layer's pages, encoded for the page kind.
// HBM-bound: every lane moves 16 bytes of page row per store, a wave covers 64/LPR whole rows per pass, rows of one
// token are consecutive in the grid so the reads of a token's heads are contiguous too.
#include "pkv_common.hpp"
#include "pkv_launch.hpp"

namespace pkv {

struct WriteArgs {
    const void* src[2];
    void* pages[2];
    float* scales[2];
    const int64_t* slots;
    const float* head_mult;
    int64_t stride_t[2], stride_h[2];
    int64_t tokens;
    int dim[2];
    int hkv;
    int heads;      // hkv (keys only) or 2 * hkv
    Div32 heads_div;
    float mult[2];
    // Rotary embedding of the key rows on their way in (rope_table null: none): cos of pair j of position p at
    // rope_table[p * dim[0] + j], sin at [p * dim[0] + dim[0] / 2 + j]; positions clamped to the table's rows.
    const float* rope_table;
    const int64_t* positions;
    int64_t rope_rows;
    int rope_interleaved;
    float rope_scale;
    // RMS norm of each key head in front of the rotation (norm_weight null: none): x / sqrt(mean(x^2) + eps) times
    // (norm_weight[i] + norm_offset), FP32 [dim[0]].
    const float* norm_weight;
    float norm_eps, norm_offset, norm_inv_dim;
};

template <int IN>
PKV_DEV float load_in(const void* base, int64_t i) {
    if constexpr (IN == CRIT_PKV_F32) return reinterpret_cast<const float*>(base)[i];
    if constexpr (IN == CRIT_PKV_BF16) return u2f((uint32_t)reinterpret_cast<const uint16_t*>(base)[i] << 16);
    return (float)reinterpret_cast<const _Float16*>(base)[i];
}

// EPL consecutive input elements of one lane as they lie in memory, fetched by 16-byte loads (the caller checked the
// alignment) and widened to FP32 only where they are used: a row waits in a quarter to half of the registers its FP32
// values would take, which is what lets twice the wavefronts be resident.
template <int IN, int EPL>
struct RawRow {
    static constexpr int N = EPL * (IN == CRIT_PKV_F32 ? 4 : 2) / 16;
    u32x4 v[N];
    PKV_DEV void load(const void* base, int64_t i) {
        const u32x4* p = reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(base) + i * (IN == CRIT_PKV_F32 ? 4 : 2));
#pragma unroll
        for (int j = 0; j < N; ++j) v[j] = __builtin_nontemporal_load(p + j);      // read once
    }
    PKV_DEV void zero() {
#pragma unroll
        for (int j = 0; j < N; ++j) v[j] = u32x4{0, 0, 0, 0};
    }
    template <int J>
    PKV_DEV float at() const {
        if constexpr (IN == CRIT_PKV_F32) {
            return u2f(v[J / 4][J % 4]);
        } else {
            const uint32_t w = v[J / 8][(J % 8) / 2];
            if constexpr (IN == CRIT_PKV_BF16) return (J & 1) ? bf16_hi(w) : bf16_lo(w);
            return (J & 1) ? f16_hi(w) : f16_lo(w);
        }
    }
    PKV_DEV void widen(float (&x)[EPL]) const {
        static_for<EPL>([&](auto j) { x[j] = at<j>(); });
    }
    // The row of the lane `delta` lanes away (xor).
    PKV_DEV RawRow across(int delta) const {
        RawRow r;
#pragma unroll
        for (int j = 0; j < N; ++j) {
            if (delta == 8) {      // (uniform) a rotation by 8 inside the row of 16 lanes: no trip through the LDS crossbar
                r.v[j] = u32x4{(unsigned)__builtin_amdgcn_update_dpp(0, (int)v[j].x, 0x128, 0xf, 0xf, true),
                               (unsigned)__builtin_amdgcn_update_dpp(0, (int)v[j].y, 0x128, 0xf, 0xf, true),
                               (unsigned)__builtin_amdgcn_update_dpp(0, (int)v[j].z, 0x128, 0xf, 0xf, true),
                               (unsigned)__builtin_amdgcn_update_dpp(0, (int)v[j].w, 0x128, 0xf, 0xf, true)};
            } else {
                r.v[j] = u32x4{(unsigned)__shfl_xor((int)v[j].x, delta), (unsigned)__shfl_xor((int)v[j].y, delta),
                               (unsigned)__shfl_xor((int)v[j].z, delta), (unsigned)__shfl_xor((int)v[j].w, delta)};
            }
        }
        return r;
    }
    // x rounded to the input type (nearest even) and packed as the row.
    PKV_DEV void pack(const float (&x)[EPL]) {
        if constexpr (IN == CRIT_PKV_F32) {
            static_for<N>([&](auto j) { v[j] = u32x4{f2u(x[4 * j]), f2u(x[4 * j + 1]), f2u(x[4 * j + 2]), f2u(x[4 * j + 3])}; });
        } else if constexpr (IN == CRIT_PKV_BF16) {
            static_for<N>([&](auto j) {
                const float x8[8] = {x[8 * j], x[8 * j + 1], x[8 * j + 2], x[8 * j + 3], x[8 * j + 4], x[8 * j + 5], x[8 * j + 6], x[8 * j + 7]};
                v[j] = pack8_bf16(x8);
            });
        } else {
            static_for<N>([&](auto j) {
                v[j] = u32x4{pack_f16(x[8 * j], x[8 * j + 1]), pack_f16(x[8 * j + 2], x[8 * j + 3]),
                             pack_f16(x[8 * j + 4], x[8 * j + 5]), pack_f16(x[8 * j + 6], x[8 * j + 7])};
            });
        }
    }
};

// 16 codes of one lane from exact divisions: the reference's arithmetic step by step, for the lanes whose quotients
// the shared-step division cannot vouch for. Four codes at a time, so the rare path needs few registers of its own.
template <int KIND, class Row>
PKV_DEV void exact_codes(const Row& row, float div, uint32_t (&w)[4]) {
    static_for<4>([&](auto k) {
        const float q[4] = {__fdiv_rn(row.template at<4 * k>(), div), __fdiv_rn(row.template at<4 * k + 1>(), div),
                            __fdiv_rn(row.template at<4 * k + 2>(), div), __fdiv_rn(row.template at<4 * k + 3>(), div)};
        uint32_t packed = 0;
        if constexpr (KIND == 3) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float r = __builtin_rintf(q[j]);            // ties to even
                r = r < -127.0f ? -127.0f : (r > 127.0f ? 127.0f : r);
                packed |= ((uint32_t)(int)r & 0xffu) << (8 * j);
            }
        } else {
            // Finite quotients: clamp, then the hardware's round-to-nearest-even conversion, two codes an instruction;
            // a NaN among the four (or infinities of both signs, whose sum is NaN too) sends them through the integer
            // encoder, which fixes the NaN code and sign and agrees with the hardware on everything else.
            const float sum = (q[0] + q[1]) + (q[2] + q[3]);
            if (sum == sum) {
                const float c0 = __builtin_amdgcn_fmed3f(q[0], -448.0f, 448.0f), c1 = __builtin_amdgcn_fmed3f(q[1], -448.0f, 448.0f);
                const float c2 = __builtin_amdgcn_fmed3f(q[2], -448.0f, 448.0f), c3 = __builtin_amdgcn_fmed3f(q[3], -448.0f, 448.0f);
                packed = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(c2, c3, __builtin_amdgcn_cvt_pk_fp8_f32(c0, c1, 0, false), true);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) packed |= e4m3_encode(q[j]) << (8 * j);
            }
        }
        w[k] = packed;
    });
}

// One row = (token, head) with head in [0, heads): keys' heads first, then values'. LPR lanes hold one row, EPL
// elements each (16 bytes of page row). KIND as in the ABI; F16: 16-bit pages are fp16, not bf16. A thread takes U rows,
// 256 / LPR apart (so a workgroup's accesses stay contiguous per pass), and issues all their loads before the first
// store. The launcher gives every thread one row: with the loads free of conditions and 46-52 registers a thread, eight
// wavefronts a SIMD are resident, and more, shorter workgroups measured faster than more rows a thread at every size
// (262,144 tokens of 8 KV heads, bf16: 389 us with one row, 397 with two, 413 with four).
// ROPE: the key rows are rotated at their tokens' positions first (the reference's rope() before write(),
// inference/fused-norms/code/torch_norms.py:89-147, over the whole head width): pairs (j, j + dim / 2) (style half: the
// partner element sits dim / 2 further, in the lane LPR / 2 away) or (2j, 2j + 1) (interleaved: both in the lane);
// a cos - b sin and b cos + a sin as separate FP32 products and a sum, rounded to the input's type as rope() rounds
// to its output's, and packed back into the row, which then goes through the append unchanged.
template <int KIND, bool F16, int IN, int LPR, int U, bool ROPE = false>
__global__ __launch_bounds__(256) void write_rows(WriteArgs a) {
    constexpr int EPL = KIND == 0 ? 8 : 16;
    constexpr int RPP = 256 / LPR;      // rows a workgroup covers per pass
    const int lane_in_row = threadIdx.x % LPR;
    // (a launch holds fewer than 2^31 rows, the launcher sees to that: 32-bit row arithmetic, and the token of a row
    // by a multiply and a shift; a 64-bit division here costs more instructions than the rest of the kernel)
    const uint32_t row0 = blockIdx.x * (uint32_t)(RPP * U) + threadIdx.x / LPR;
    const uint32_t n_rows = (uint32_t)(a.tokens * a.heads);
    const int i0 = lane_in_row * EPL;
    RawRow<IN, EPL> raw[U];
    int64_t slot[U];
    int head[U];
    bool second[U], in[U], live[U];      // second: a row of the values; live: this lane holds elements of the row
    float mult[U];                       // "fp8" pages: the row's divisor, fetched with its inputs
    int64_t rope_pos = 0;                // ROPE: the token's position, fetched with its inputs (the table's row waits for it)
    // Every load of the U rows is issued before anything waits for one: no load sits under a condition (a row past the
    // end reads row 0, a lane past a narrow row's width reads the row's start) and nothing indexes the launch arguments
    // by a value a lane computes (which would fetch them from memory): the choice between the keys' and the values'
    // arguments is a select between scalars.
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t row = row0 + u * RPP;
        in[u] = row < n_rows;
        const uint32_t rowc = in[u] ? row : 0;
        const uint32_t t = div32(a.heads_div, rowc);
        const int h = (int)(rowc - t * (uint32_t)a.heads);
        second[u] = h >= a.hkv;
        head[u] = second[u] ? h - a.hkv : h;
        live[u] = in[u] && i0 < (second[u] ? a.dim[1] : a.dim[0]);
        slot[u] = a.slots[t];
        mult[u] = second[u] ? a.mult[1] : a.mult[0];
        if constexpr (KIND == 1) {
            if (a.head_mult) mult[u] = a.head_mult[(second[u] ? a.hkv : 0) + head[u]];
        }
        const void* src = second[u] ? a.src[1] : a.src[0];
        const int64_t st = second[u] ? a.stride_t[1] : a.stride_t[0], sh = second[u] ? a.stride_h[1] : a.stride_h[0];
        raw[u].load(src, (int64_t)t * st + head[u] * sh + (live[u] ? i0 : 0));
        if constexpr (ROPE) rope_pos = a.positions[t];
    }
    __builtin_amdgcn_sched_barrier(0);      // (nothing that waits for a load moves up among the loads)
    if constexpr (ROPE) {
        static_assert(U == 1 && LPR >= 2, "one row a thread, a row over two lanes or more");
        int64_t pos = rope_pos;
        pos = pos < 0 ? 0 : (pos > a.rope_rows - 1 ? a.rope_rows - 1 : pos);
        const int half = a.dim[0] >> 1;
        const bool upper = lane_in_row >= LPR / 2;
        // (every lane takes part in the exchange and loads a row of the table: a values' row is left as it was)
        const int j0 = a.rope_interleaved ? i0 >> 1 : (upper ? i0 - half : i0);
        constexpr int PAIRS = EPL;      // style half: one pair an element; interleaved: EPL / 2 pairs
        float cs[PAIRS], sn[PAIRS];
        // (16-byte loads: the table's rows and a lane's first pair are multiples of four floats)
        const float4* line = reinterpret_cast<const float4*>(a.rope_table + pos * a.dim[0] + j0);
        const float4* line_sin = reinterpret_cast<const float4*>(a.rope_table + pos * a.dim[0] + half + j0);
        const int quads = a.rope_interleaved ? EPL / 8 : EPL / 4;
#pragma unroll
        for (int j = 0; j < PAIRS / 4; ++j) {
            const float4 c = j < quads ? line[j] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            const float4 z = j < quads ? line_sin[j] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            cs[4 * j] = c.x, cs[4 * j + 1] = c.y, cs[4 * j + 2] = c.z, cs[4 * j + 3] = c.w;
            sn[4 * j] = z.x, sn[4 * j + 1] = z.y, sn[4 * j + 2] = z.z, sn[4 * j + 3] = z.w;
        }
        if (a.rope_scale != 1.0f) {
#pragma unroll
            for (int j = 0; j < PAIRS; ++j) cs[j] = cs[j] * a.rope_scale, sn[j] = sn[j] * a.rope_scale;
        }
        float mine[EPL], other[EPL], y[EPL];
        raw[0].widen(mine);
        if (!a.norm_weight) raw[0].across(LPR / 2).widen(other);
        if (a.norm_weight) {
            // The reference's rms_norm_rope (inference/fused-norms/code/torch_norms.py:149-176): each head normalised
            // in FP32, times its weight, rotated, one rounding at the end. The sum of squares in a fixed order, the same
            // for every page kind: squares rounded one by one, groups of 8 consecutive elements summed in order, the
            // groups by a balanced tree of adjacent pairs (a lane of 16 elements adds its two groups first; then the
            // row's lanes 1, 2, 4 ... apart); mean, square root and reciprocal correctly rounded.
            float sq = 0.0f;
#pragma unroll
            for (int g8 = 0; g8 < EPL / 8; ++g8) {
                float s8 = mine[8 * g8] * mine[8 * g8];
#pragma unroll
                for (int j = 1; j < 8; ++j) s8 = s8 + mine[8 * g8 + j] * mine[8 * g8 + j];
                sq = g8 == 0 ? s8 : sq + s8;
            }
            sq = LPR > 1 ? group_sum<(LPR > 1 ? LPR : 2)>(sq) : sq;      // (the butterfly's sums, lane pairs met in the vector pipe)
            const float mean = sq * a.norm_inv_dim;      // (the width is a power of two: the product is the quotient, exactly)
            // __builtin_sqrtf is the correctly rounded root (hipcc's default for sqrtf and "/"); __fsqrt_rn is not,
            // unless OCML_BASIC_ROUNDED_OPERATIONS is defined: it is the hardware's approximate one.
            const float r = __fdiv_rn(1.0f, __builtin_sqrtf(mean + a.norm_eps));
            const float4* w_mine = reinterpret_cast<const float4*>(a.norm_weight + i0);
#pragma unroll
            for (int j = 0; j < EPL / 4; ++j) {
                const float4 wm = w_mine[j];
                const float m4[4] = {wm.x, wm.y, wm.z, wm.w};
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float fm = a.norm_offset != 0.0f ? m4[k] + a.norm_offset : m4[k];
                    mine[4 * j + k] = (mine[4 * j + k] * r) * fm;
                }
            }
            // the partner lane's elements (style half) as that lane normalised them: the same operations on the same
            // numbers as normalising them here, without doing it twice
#pragma unroll
            for (int j = 0; j < EPL; ++j) {
                if (LPR / 2 == 8) other[j] = u2f((uint32_t)__builtin_amdgcn_update_dpp(0, (int)f2u(mine[j]), 0x128, 0xf, 0xf, true));
                else other[j] = __shfl_xor(mine[j], LPR / 2);
            }
        }
        if (a.rope_interleaved) {
#pragma unroll
            for (int j = 0; j < EPL / 2; ++j) {
                const float x0 = mine[2 * j], x1 = mine[2 * j + 1];
                y[2 * j] = x0 * cs[j] - x1 * sn[j];
                y[2 * j + 1] = x1 * cs[j] + x0 * sn[j];
            }
        } else {
            {
                // (a - b is a + (-b), bit for bit: the lower half's sign goes into its sines, one XOR an element, and
                // the two halves run the same three operations)
                const uint32_t flip = upper ? 0u : 0x80000000u;
#pragma unroll
                for (int j = 0; j < EPL; ++j) y[j] = mine[j] * cs[j] + other[j] * u2f(f2u(sn[j]) ^ flip);
            }
        }
        if (!second[0]) raw[0].pack(y);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        // (a whole row's lanes agree on these, so the row-scale exchange below stays among participating lanes)
        if (!in[u] || slot[u] < 0) continue;
        if constexpr (KIND >= 2) {
            if (!live[u]) raw[u].zero();      // the row's maximum is over its own elements
        }
        float x[EPL];
        raw[u].widen(x);
        const int dim = second[u] ? a.dim[1] : a.dim[0];
        void* const pages = second[u] ? a.pages[1] : a.pages[0];
        float* const scales = second[u] ? a.scales[1] : a.scales[0];
        const int64_t dst = (slot[u] * a.hkv + head[u]) * dim + i0;
        if constexpr (KIND == 0) {
            uint4 v;
            if constexpr ((IN == CRIT_PKV_BF16 && !F16) || (IN == CRIT_PKV_F16 && F16)) {
                // the pages' type is the inputs' own: the row as it came, bit for bit (torch's .to() of a tensor's own
                // dtype is the tensor: a NaN keeps its payload, where a cast from another type stores the canonical one)
                v = make_uint4(raw[u].v[0].x, raw[u].v[0].y, raw[u].v[0].z, raw[u].v[0].w);
            } else if constexpr (F16) {
                v = make_uint4(pack_f16(x[0], x[1]), pack_f16(x[2], x[3]), pack_f16(x[4], x[5]), pack_f16(x[6], x[7]));
            } else {
                const u32x4 packed = pack8_bf16(x);
                v = make_uint4(packed.x, packed.y, packed.z, packed.w);
            }
            if (live[u]) __builtin_nontemporal_store(u32x4{v.x, v.y, v.z, v.w}, reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(pages) + dst));
        } else {
            float div;
            bool zero_row = false;
            if constexpr (KIND == 1) {
                div = mult[u];
            } else {
                float amax = 0.0f;
#pragma unroll
                for (int j = 0; j < EPL; ++j) {
                    const float m = __builtin_fabsf(x[j]);
                    amax = (m > amax || m != m) ? m : amax;       // a NaN in the row makes the scale NaN, as torch's amax
                }
#pragma unroll
                for (int o = 1; o < LPR; o <<= 1) {
                    const float other = __shfl_xor(amax, o);
                    amax = (other > amax || other != other) ? other : amax;
                }
                const float top = KIND == 2 ? 448.0f : 127.0f;
                div = __fdiv_rn(amax, top);
                div = div < 1e-30f ? 1e-30f : div;               // clamp(min=1e-30); NaN stays NaN
                zero_row = amax == 0.0f;
                if (lane_in_row == 0) scales[slot[u] * a.hkv + head[u]] = div;
            }
            // The quotients by the shared steps of one division, straight through to the codes; where the divisor does
            // not allow that (an all-zero row's does, the 1e-30 floor: its quotients are zeros of the inputs' signs
            // either way) or a quotient came out NaN (a NaN or infinite input, a quotient past FP32), the lane's codes
            // are made again from exact divisions.
            uint32_t w[4];
            const Quotients quot(div);
            bool coded = quot.plain || zero_row;
            float sum = 0.0f;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                float c[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float q = quot.of(x[4 * k + j]);
                    if constexpr (KIND == 3) {
                        c[j] = __builtin_amdgcn_fmed3f(__builtin_rintf(q), -127.0f, 127.0f);      // ties to even
                    } else {
                        if constexpr (KIND == 1) sum += q;      // (a row's own scale keeps its quotients finite)
                        c[j] = __builtin_amdgcn_fmed3f(q, -448.0f, 448.0f);
                    }
                }
                if constexpr (KIND == 3) {
                    w[k] = ((uint32_t)(int)c[0] & 0xffu) | (((uint32_t)(int)c[1] & 0xffu) << 8) | (((uint32_t)(int)c[2] & 0xffu) << 16) |
                           ((uint32_t)(int)c[3] << 24);
                } else {
                    int packed = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], 0, false);
                    w[k] = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], packed, true);
                }
                // (four independent chains are enough to fill the pipeline; interleaving all sixteen costs the registers
                // of two more resident wavefronts)
                __builtin_amdgcn_sched_barrier(0);
            }
            coded = coded && sum == sum;
            if (__builtin_expect(!coded, 0)) exact_codes<KIND>(raw[u], div, w);
            if (live[u]) __builtin_nontemporal_store(u32x4{w[0], w[1], w[2], w[3]}, reinterpret_cast<u32x4*>(reinterpret_cast<uint8_t*>(pages) + dst));
        }
    }
}

// Any width and alignment: one lane per row element group of one (scalar loads and stores); the row scale by a
// loop. Used when a row is not a whole number of 16-byte lanes or a stride breaks the alignment.
template <int KIND, bool F16, int IN>
__global__ __launch_bounds__(256) void write_rows_scalar(WriteArgs a) {
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row >= a.tokens * a.heads) return;
    const int64_t t = row / a.heads;
    int head = (int)(row % a.heads);
    const int which = head >= a.hkv ? 1 : 0;
    head -= which * a.hkv;
    const int64_t slot = a.slots[t];
    if (slot < 0) return;
    const int dim = a.dim[which];
    const int64_t src = t * a.stride_t[which] + head * a.stride_h[which];
    const int64_t dst = (slot * a.hkv + head) * dim;
    float div = 1.0f;
    if constexpr (KIND == 1) div = a.head_mult ? a.head_mult[which * a.hkv + head] : a.mult[which];
    if constexpr (KIND >= 2) {
        float amax = 0.0f;
        for (int i = 0; i < dim; ++i) {
            const float m = __builtin_fabsf(load_in<IN>(a.src[which], src + i));
            amax = (m > amax || m != m) ? m : amax;
        }
        div = __fdiv_rn(amax, KIND == 2 ? 448.0f : 127.0f);
        div = div < 1e-30f ? 1e-30f : div;
        a.scales[which][slot * a.hkv + head] = div;
    }
    for (int i = 0; i < dim; ++i) {
        const float x = load_in<IN>(a.src[which], src + i);
        if constexpr (KIND == 0 && ((IN == CRIT_PKV_BF16 && !F16) || (IN == CRIT_PKV_F16 && F16))) {
            // (the inputs' own type: the element's bits as they came)
            reinterpret_cast<uint16_t*>(a.pages[which])[dst + i] = reinterpret_cast<const uint16_t*>(a.src[which])[src + i];
        } else if constexpr (KIND == 0) {
            reinterpret_cast<uint16_t*>(a.pages[which])[dst + i] = (uint16_t)(F16 ? f16_bits(x) : bf16_rne(x));
        } else {
            const float q = __fdiv_rn(x, div);
            uint32_t code;
            if constexpr (KIND == 3) {
                float r = __builtin_rintf(q);
                r = r < -127.0f ? -127.0f : (r > 127.0f ? 127.0f : r);
                code = (uint32_t)(int)r & 0xffu;
            } else {
                code = e4m3_encode(q);
            }
            reinterpret_cast<uint8_t*>(a.pages[which])[dst + i] = (uint8_t)code;
        }
    }
}

template <int KIND, bool F16, int IN>
static int launch_kind(const WriteArgs& a, int lpr, bool vector, hipStream_t stream) {
    if (!vector) {
        if (a.rope_table) return CRIT_PKV_E_GEOMETRY;      // (the rotation lives in the vector kernel)
        const int64_t blocks = (a.tokens * a.heads + 255) / 256;
        hipLaunchKernelGGL((write_rows_scalar<KIND, F16, IN>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
        return hip_code(hipGetLastError());
    }
    // The vector kernels count rows in 32 bits: more tokens than 2^31 rows hold go in several launches.
    const int64_t most = (((int64_t)1 << 31) - (1 << 16)) / a.heads;
    if (a.tokens > most) {
        const int in_bytes = IN == CRIT_PKV_F32 ? 4 : 2;
        for (int64_t t0 = 0; t0 < a.tokens; t0 += most) {
            WriteArgs part = a;
            part.tokens = a.tokens - t0 < most ? a.tokens - t0 : most;
            part.slots = a.slots + t0;
            if (a.positions) part.positions = a.positions + t0;
            for (int w = 0; w < 2; ++w) {
                if (a.src[w]) part.src[w] = reinterpret_cast<const char*>(a.src[w]) + t0 * a.stride_t[w] * in_bytes;
            }
            const int code = launch_kind<KIND, F16, IN>(part, lpr, vector, stream);
            if (code) return code;
        }
        return 0;
    }
    const int64_t rows = a.tokens * a.heads;
    const int rows_per_block = 256 / lpr;
    const int64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
    if (a.rope_table) {      // (head widths 64, 128 and 256: 4 to 32 lanes a row)
        switch (lpr) {
#define PKV_CASE(L)                                                                                                 \
    case L:                                                                                                         \
        hipLaunchKernelGGL((write_rows<KIND, F16, IN, L, 1, true>), dim3((unsigned)blocks), dim3(256), 0, stream, a); \
        break;
            PKV_CASE(4) PKV_CASE(8) PKV_CASE(16) PKV_CASE(32)
#undef PKV_CASE
            default:
                return CRIT_PKV_E_GEOMETRY;
        }
        return hip_code(hipGetLastError());
    }
    switch (lpr) {
#define PKV_CASE(L)                                                                                                 \
    case L:                                                                                                         \
        hipLaunchKernelGGL((write_rows<KIND, F16, IN, L, 1>), dim3((unsigned)blocks), dim3(256), 0, stream, a);       \
        break;
        PKV_CASE(1) PKV_CASE(2) PKV_CASE(4) PKV_CASE(8) PKV_CASE(16) PKV_CASE(32) PKV_CASE(64)
#undef PKV_CASE
        default:
            return CRIT_PKV_E_GEOMETRY;
    }
    return hip_code(hipGetLastError());
}

template <int KIND, bool F16>
static int launch_in(const WriteArgs& a, int in_dtype, int lpr, bool vector, hipStream_t stream) {
    switch (in_dtype) {
        case CRIT_PKV_F32: return launch_kind<KIND, F16, CRIT_PKV_F32>(a, lpr, vector, stream);
        case CRIT_PKV_BF16: return launch_kind<KIND, F16, CRIT_PKV_BF16>(a, lpr, vector, stream);
        case CRIT_PKV_F16: return launch_kind<KIND, F16, CRIT_PKV_F16>(a, lpr, vector, stream);
    }
    return CRIT_PKV_E_DTYPE;
}

static int next_pow2(int n) {
    int p = 1;
    while (p < n) p <<= 1;
    return p;
}

int launch_write(const crit_pkv_write_params* p, hipStream_t stream) {
    if (!p || !p->keys || !p->key_pages || !p->slots) return CRIT_PKV_E_NULL;
    if ((p->values == nullptr) != (p->value_pages == nullptr)) return CRIT_PKV_E_NULL;
    if (p->tokens < 0 || p->kv_heads < 1 || p->head_dim < 1 || (p->values && p->value_dim < 1)) return CRIT_PKV_E_GEOMETRY;
    if (p->kind < 0 || p->kind > 3) return CRIT_PKV_E_DTYPE;
    if (p->kind >= 2 && (!p->key_scales || (p->values && !p->value_scales))) return CRIT_PKV_E_NULL;
    if (p->kind == 0 && p->page_dtype != CRIT_PKV_BF16 && p->page_dtype != CRIT_PKV_F16) return CRIT_PKV_E_DTYPE;
    if (p->tokens == 0) return 0;
    WriteArgs a;
    a.src[0] = p->keys, a.src[1] = p->values;
    a.pages[0] = p->key_pages, a.pages[1] = p->value_pages;
    a.scales[0] = p->key_scales, a.scales[1] = p->value_scales;
    a.slots = p->slots;
    a.head_mult = p->kind == 1 ? p->head_multipliers : nullptr;
    a.stride_t[0] = p->key_stride_t, a.stride_t[1] = p->value_stride_t;
    a.stride_h[0] = p->key_stride_h, a.stride_h[1] = p->value_stride_h;
    a.tokens = p->tokens;
    a.dim[0] = p->head_dim, a.dim[1] = p->values ? p->value_dim : p->head_dim;
    a.hkv = p->kv_heads;
    a.heads = p->values ? 2 * p->kv_heads : p->kv_heads;
    a.heads_div = make_div32((uint32_t)a.heads);
    a.mult[0] = p->key_multiplier, a.mult[1] = p->value_multiplier;
    a.rope_table = p->rope_table, a.positions = p->rope_positions, a.rope_rows = p->rope_rows;
    a.rope_interleaved = p->rope_interleaved ? 1 : 0, a.rope_scale = p->rope_scale;
    a.norm_weight = p->norm_weight, a.norm_eps = p->norm_eps, a.norm_offset = p->norm_offset;
    a.norm_inv_dim = 1.0f / (float)p->head_dim;
    if (p->norm_weight && (!p->rope_table || (reinterpret_cast<uintptr_t>(p->norm_weight) % 16))) return CRIT_PKV_E_GEOMETRY;
    if (p->rope_table) {
        // the whole head width rotates, a power of two of whole lanes; the lanes of a values' row of another width
        // would not line up with the keys' in the exchange
        if (!p->rope_positions) return CRIT_PKV_E_NULL;
        if (p->rope_rows < 1 || (p->head_dim != 64 && p->head_dim != 128 && p->head_dim != 256) ||
            (p->values && p->value_dim > p->head_dim) || (reinterpret_cast<uintptr_t>(p->rope_table) % 16))
            return CRIT_PKV_E_GEOMETRY;
    }
    // The vector path: rows are whole 16-byte lanes on both sides and every row start is 16-byte aligned.
    const int epl = p->kind == 0 ? 8 : 16;
    const int in_bytes = p->in_dtype == CRIT_PKV_F32 ? 4 : 2;
    const int in_align = 16 / in_bytes;
    const int widest = a.dim[0] > a.dim[1] ? a.dim[0] : a.dim[1];
    const int lpr = next_pow2((widest + epl - 1) / epl);
    bool vector = lpr <= 64;
    for (int w = 0; w < (p->values ? 2 : 1); ++w) {
        vector = vector && a.dim[w] % epl == 0 && a.stride_t[w] % in_align == 0 && a.stride_h[w] % in_align == 0 &&
                 (reinterpret_cast<uintptr_t>(a.src[w]) % 16) == 0 && (reinterpret_cast<uintptr_t>(a.pages[w]) % 16) == 0;
    }
    const bool f16 = p->kind == 0 && p->page_dtype == CRIT_PKV_F16;
    switch (p->kind) {
        case 0: return f16 ? launch_in<0, true>(a, p->in_dtype, lpr, vector, stream)
                           : launch_in<0, false>(a, p->in_dtype, lpr, vector, stream);
        case 1: return launch_in<1, false>(a, p->in_dtype, lpr, vector, stream);
        case 2: return launch_in<2, false>(a, p->in_dtype, lpr, vector, stream);
        case 3: return launch_in<3, false>(a, p->in_dtype, lpr, vector, stream);
    }
    return CRIT_PKV_E_DTYPE;
}

}   // namespace pkv
