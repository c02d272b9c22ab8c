// Device helpers shared by the paged-KV kernels (gfx950 only): 16-bit float bit casts, the E4M3FN codec, DPP
// reductions inside a 16-lane row, and the online-softmax fold.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>
#include <utility>

#include "../../include/crit_pkv.h"

namespace pkv {

// Native vectors for values that live in register arrays: the compiler promotes arrays of these to registers, which
// it does not always do for arrays of the runtime's uint4 / uint2 classes copied whole.
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;

#define PKV_DEV __device__ __forceinline__

// A loop unrolled by template expansion: f(std::integral_constant<int, 0>{}), ..., f(<N - 1>). Register arrays indexed
// through it are indexed by constants whatever the optimiser makes of the body.
template <class F, int... I>
PKV_DEV void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
PKV_DEV void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

PKV_DEV uint32_t f2u(float x) { return __builtin_bit_cast(uint32_t, x); }
PKV_DEV float u2f(uint32_t x) { return __builtin_bit_cast(float, x); }

// -- division by a value fixed per launch ------------------------------------------------------------------------------------
// n / d for 0 <= n < 2^31 by a multiply and a shift (d >= 1): l = ceil(log2 d), magic = floor(2^32 (2^l - d) / d) + 1.
struct Div32 {
    uint32_t magic, shift;
};
inline Div32 make_div32(uint32_t d) {
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;
    return {(uint32_t)((((1ull << l) - (uint64_t)d) << 32) / (uint64_t)d + 1), l};
}
PKV_DEV uint32_t div32(Div32 m, uint32_t n) { return (__umulhi(m.magic, n) + n) >> m.shift; }

// x / d, correctly rounded, for many x and one d: the steps of the compiler's own FP32 division (a reciprocal refined
// once, the quotient refined twice through exact residuals) with everything that depends on d alone computed once.
// Those steps give the correctly rounded quotient wherever none of them overflows or loses bits to underflow, which
// `plain` guarantees for the quotients a page code can tell apart (|x / d| from 2^-12 up, below 2^127): d in
// 2^-60 .. 2^60, where the reciprocal, the residuals of such quotients (2^-24 of x) and their products stay normal.
// Smaller quotients may come out a few steps off and still round to the same (zero) code; a quotient that overflows
// comes out NaN, which the callers send through the exact division. The residuals are taken negated, d q - x, and
// subtracted: the same bits, and a zero x keeps its sign through every step (-0 + +0 would be +0).
struct Quotients {
    float d, r;
    bool plain;
    PKV_DEV explicit Quotients(float div) : d(div) {
        plain = div >= 0x1p-60f && div <= 0x1p60f;
        const float r0 = __builtin_amdgcn_rcpf(div);
        r = __builtin_fmaf(__builtin_fmaf(-div, r0, 1.0f), r0, r0);
    }
    PKV_DEV float of(float x) const {
        float q = x * r;
        q = __builtin_fmaf(-__builtin_fmaf(d, q, -x), r, q);
        q = __builtin_fmaf(-__builtin_fmaf(d, q, -x), r, q);
        return q;
    }
};

// -- bf16 / f16 ---------------------------------------------------------------------------------------------------------
PKV_DEV float bf16_lo(uint32_t w) { return u2f(w << 16); }
PKV_DEV float bf16_hi(uint32_t w) { return u2f(w & 0xffff0000u); }

// FP32 -> BF16 bits, round to nearest even; NaN -> 0xFFFF: what torch's CPU cast of a tensor stores (its vectorised
// conversion, AVX2 and AVX-512 alike, blends 0xFFFF in for every NaN; its scalar conversion, which only a build
// without those reaches, returns 0x7FC0: the reference's stored bytes for a NaN follow the host it runs on).
PKV_DEV uint32_t bf16_rne(float x) {
    uint32_t u = f2u(x);
    uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    return (x != x) ? 0xffffu : r;
}
PKV_DEV uint32_t pack_bf16(float a, float b) { return bf16_rne(a) | (bf16_rne(b) << 16); }
// Eight FP32 values as four BF16 pairs with the same bits as pack_bf16, by the hardware's conversion (v_cvt_pk_bf16_f32:
// round to nearest even, like bf16_rne, for every number) where no value is a NaN, which one test over the packed
// words decides (a 16-bit half above 0x7F80 in magnitude): a NaN comes out of the hardware quiet but with its payload,
// and torch's cast stores 0xFFFF, so then the words are made again one value at a time.
PKV_DEV u32x4 pack8_bf16(const float (&x)[8]) {
    typedef __attribute__((ext_vector_type(2))) __bf16 pair_t;
    uint32_t w[4], any = 0u;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const pair_t r = {(__bf16)x[2 * j], (__bf16)x[2 * j + 1]};
        w[j] = __builtin_bit_cast(uint32_t, r);
        any |= (w[j] & 0x7fff7fffu) + 0x007f007fu;
    }
    if (any & 0x80008000u) {
#pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = pack_bf16(x[2 * j], x[2 * j + 1]);
    }
    return u32x4{w[0], w[1], w[2], w[3]};
}

PKV_DEV float f16_lo(uint32_t w) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu)); }
PKV_DEV float f16_hi(uint32_t w) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16)); }
PKV_DEV uint32_t f16_bits(float x) { return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)x); }   // RNE
PKV_DEV uint32_t pack_f16(float a, float b) { return f16_bits(a) | (f16_bits(b) << 16); }

// -- E4M3FN -------------------------------------------------------------------------------------------------------------
// FP32 -> code: clamp to [-448, 448], round to nearest code, ties to even; sign from the sign bit (-0.0 -> 0x80);
// NaN -> 0x7F | sign. Integer arithmetic only, so the bytes do not depend on any conversion mode of the hardware.
PKV_DEV uint32_t e4m3_encode(float x) {
    const uint32_t bits = f2u(x);
    const uint32_t sign = (bits >> 24) & 0x80u;
    float a = __builtin_fabsf(x);
    const bool nan = x != x;
    a = a > 448.0f ? 448.0f : a;
    const uint32_t ab = f2u(a);
    int ex = (int)(ab >> 23) - 127;
    int sex = ex < -126 ? -126 : ex;
    const float frac = a * u2f((uint32_t)(127 - sex) << 23);               // exact scaling into [1, 2)
    int mant = (int)__builtin_rintf((frac - 1.0f) * 8.0f);                  // ties to even
    const bool carry = mant == 8;
    ex = carry ? ex + 1 : ex;
    mant = carry ? 0 : mant;
    const uint32_t normal = ((uint32_t)(ex + 7) << 3) | (uint32_t)mant;
    const uint32_t sub = (uint32_t)(int)__builtin_rintf(a * 512.0f);       // below 2^-6: multiples of 2^-9
    uint32_t code = a < 0.015625f ? sub : normal;
    code = nan ? 0x7fu : code;
    return code | sign;
}

// Two E4M3FN codes (bytes 0,1 or 2,3 of w) -> FP32, by the hardware conversion (OCP E4M3 on gfx950).
template <bool HI>
PKV_DEV f32x2 e4m3_pair(uint32_t w) { return __builtin_amdgcn_cvt_pk_f32_fp8((int)w, HI); }

// -- cross-lane ------------------------------------------------------------------------------------------------------------
// DPP controls: quad_perm [1,0,3,2] = 0xB1 (xor 1), quad_perm [2,3,0,1] = 0x4E (xor 2), row_half_mirror = 0x141
// (lane i <-> 7 - i inside each 8), row_mirror = 0x140 (lane i <-> 15 - i inside each 16).
template <int CTRL>
PKV_DEV float dpp(float x) {
    return u2f((uint32_t)__builtin_amdgcn_update_dpp(0, (int)f2u(x), CTRL, 0xf, 0xf, true));
}

// A lane's value and that of lane ^ 16 (ROWS false) or lane ^ 32 (true), in an order that depends on the lane: for
// operations that commute. One lane swap in the vector pipe (v_permlane16_swap / v_permlane32_swap), where a shuffle
// is a round trip through the LDS crossbar.
struct Met {
    float a, b;
};
template <bool HALVES>
PKV_DEV Met meet(float x) {
    const int v = (int)f2u(x);
    if constexpr (HALVES) {
        const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
        return Met{u2f((uint32_t)r[0]), u2f((uint32_t)r[1])};
    } else {
        const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
        return Met{u2f((uint32_t)r[0]), u2f((uint32_t)r[1])};
    }
}

// The same for lane ^ O, any power of two: a rotation inside the row of 16 for 8, a shuffle below that.
template <int O>
PKV_DEV Met meet_at(float x) {
    if constexpr (O == 32) return meet<true>(x);
    else if constexpr (O == 16) return meet<false>(x);
    else if constexpr (O == 8) return Met{x, u2f((uint32_t)__builtin_amdgcn_update_dpp(0, (int)f2u(x), 0x128, 0xf, 0xf, true))};      // row_ror:8
    else return Met{x, __shfl_xor(x, O)};
}
// Sum / maximum over the lanes that hold the same place in each group of LPR lanes of the wavefront (a butterfly: every
// lane ends with the same bits).
template <int LPR>
PKV_DEV float sum_over_groups(float x) {
    if constexpr (LPR < 64) {
        const Met m = meet_at<LPR>(x);
        return sum_over_groups<LPR * 2>(m.a + m.b);
    } else {
        return x;
    }
}
template <int LPR>
PKV_DEV float max_over_groups(float x) {
    if constexpr (LPR < 64) {
        const Met m = meet_at<LPR>(x);
        return max_over_groups<LPR * 2>(__builtin_fmaxf(m.a, m.b));
    } else {
        return x;
    }
}

// The sum of x over the lanes up to and including this one of the wavefront, by data-parallel-primitive adds (shifts
// of 1, 2, 4, 8 inside each row of 16 lanes, then lane 15 of a row to the next row, lane 31 to the upper half): six
// vector instructions where a shuffle through the LDS crossbar is a round trip each.
PKV_DEV unsigned wave_inclusive_sum(unsigned x) {
    int v = (int)x;
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);      // row_shr:1 (zeros shifted in)
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);      // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);      // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);      // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);     // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);     // row_bcast:31 into rows 2 and 3
    return (unsigned)v;
}

// Sum over the LANES (2 to 64, a power of two) lanes of each aligned group; every lane gets the same bits.
template <int LANES>
PKV_DEV float group_sum(float x) {
    x += dpp<0xB1>(x);
    if constexpr (LANES >= 4) x += dpp<0x4E>(x);
    if constexpr (LANES >= 8) x += dpp<0x141>(x);
    if constexpr (LANES >= 16) x += dpp<0x140>(x);
    if constexpr (LANES >= 32) {
        const Met m = meet<false>(x);
        x = m.a + m.b;
    }
    if constexpr (LANES >= 64) {
        const Met m = meet<true>(x);
        x = m.a + m.b;
    }
    return x;
}
template <int LANES>
PKV_DEV float group_max(float x) {
    x = __builtin_fmaxf(x, dpp<0xB1>(x));
    if constexpr (LANES >= 4) x = __builtin_fmaxf(x, dpp<0x4E>(x));
    if constexpr (LANES >= 8) x = __builtin_fmaxf(x, dpp<0x141>(x));
    if constexpr (LANES >= 16) x = __builtin_fmaxf(x, dpp<0x140>(x));
    if constexpr (LANES >= 32) {
        const Met m = meet<false>(x);
        x = __builtin_fmaxf(m.a, m.b);
    }
    if constexpr (LANES >= 64) {
        const Met m = meet<true>(x);
        x = __builtin_fmaxf(m.a, m.b);
    }
    return x;
}

// -- online softmax, base 2 -----------------------------------------------------------------------------------------------
PKV_DEV float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }   // v_exp_f32; exp2(-inf) = 0

// A partial state (m, l) into the running one, in the caller's order: out = out * keep + partial * take.
struct Fold {
    float m, l, keep, take;
};
PKV_DEV Fold fold(float m_run, float l_run, float m, float l) {
    Fold f;
    f.m = __builtin_fmaxf(m_run, m);
    const float sub = f.m == -INFINITY ? 0.0f : f.m;
    f.keep = exp2_fast(m_run - sub);
    f.take = exp2_fast(m - sub);
    f.l = __builtin_fmaf(l_run, f.keep, l * f.take);
    return f;
}

PKV_DEV void store_out(void* out, int dtype, int64_t index, float x) {
    if (dtype == CRIT_PKV_BF16) {
        reinterpret_cast<uint16_t*>(out)[index] = (uint16_t)bf16_rne(x);
    } else if (dtype == CRIT_PKV_F16) {
        reinterpret_cast<uint16_t*>(out)[index] = (uint16_t)f16_bits(x);
    } else {
        reinterpret_cast<float*>(out)[index] = x;
    }
}

inline int hip_code(hipError_t e) { return e == hipSuccess ? 0 : (int)e; }

}   // namespace pkv
