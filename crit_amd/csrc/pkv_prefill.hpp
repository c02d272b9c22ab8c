// Declarations of the chunked-prefill kernel: the launch arguments, the MFMA wrappers, the LDS swizzle of V^T, the
// order in which chunks are taken.
#pragma once
#include "pkv_common.hpp"

namespace pkv {

struct PrefillArgs {
    const uint8_t* q;
    const uint8_t* kp;
    const uint8_t* vp;
    const float* ks;
    const float* vs;
    const float* hm;
    const int32_t* tables;
    const int64_t* tables64;
    const int32_t* table_rows;
    const int32_t* starts;
    const int32_t* counts;
    const int64_t* positions;
    void* out;
    float* lse;
    const float* sinks;
    int64_t q_st, q_sh, o_st, o_sh, tab_stride;
    int tab_width, chunks, max_count, hq, hkv, g, page, page_l, sliding, out_dtype, tiles;
    uint32_t page_magic;     // n / page == (mulhi(page_magic, n) + n) >> page_l for 0 <= n < 2^31
    float sscale, k_mult, v_mult;
    // A chunk whose own positions from `first` on are read from fresh 16-bit rows takes two launches that hand a row's
    // running state (unnormalised output, maximum, sum) through `state`: mode 1 reads the positions below the chunk's
    // first fresh one from the pages and writes the state; mode 2 starts from it, reads the positions from the first
    // fresh one on as rows of kp / vp (row = the chunk's first token + position - the chunk's position, no page table) and
    // finishes the rows. Mode 0: one launch over the pages.
    const int64_t* firsts;   // [chunks], or null: the chunk's position (all of its own positions are fresh)
    float* state;            // [token][head][kStateRow] FP32
    int mode;
    int iqk;                 // INT8 pages: integer scores from INT8 query codes (the reference's int8_qk)
    uint32_t k_slot_bytes, v_slot_bytes;     // bytes from one slot's (or fresh row's) K / V row to the next
};
constexpr int kStatePad = 4;      // a row of the state is head_dim + 4 floats: the output, the maximum, the sum, 16-byte rows

// A wavefront raises its priority while it issues matrix instructions, so the other wavefront of its SIMD fills the
// gaps with vector work instead of delaying them.
#define PKV_PRIO(x) __builtin_amdgcn_s_setprio(x)
// Nothing is scheduled across this point: it fixes the order of the phases the kernel lays out by hand.
#define PKV_SB() __builtin_amdgcn_sched_barrier(0)
// The running maximum a row's exponentials are taken against moves only when a block's maximum exceeds it by more
// than this (in log2 units): probabilities then reach 2^8 at most, far inside the range of the 16-bit operand and the
// FP32 sums, the final division by the row's sum (taken against the same reference) cancels the factor, and the
// accumulators are rescaled on a handful of blocks instead of most of them. A row's own data decide, nothing else.
constexpr float kMaxSlack = 8.0f;
constexpr int BM = 128;   // query rows a workgroup holds
constexpr int BN = 64;    // keys a block holds

template <bool F16>
PKV_DEV f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    if constexpr (F16) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
}
template <bool F16>
PKV_DEV f32x16 mfma(u32x4 a, uint4 b, f32x16 c) { return mfma<F16>(a, u32x4{b.x, b.y, b.z, b.w}, c); }
template <bool F16>
PKV_DEV f32x16 mfma(uint4 a, uint4 b, f32x16 c) {
    if constexpr (F16) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
}

// Two probabilities as a 16-bit pair by the hardware conversions (round to nearest even).
template <bool F16>
PKV_DEV uint32_t to_pair(float a, float b) {
    if constexpr (F16) return pack_f16(a, b);
    typedef __attribute__((ext_vector_type(2))) __bf16 pair_t;
    pair_t r = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(uint32_t, r);
}

// Two codes (bytes 0,1 or 2,3 of a word of E4M3 or INT8 codes) -> two BF16 values in one word, exactly.
template <int KIND, bool HI>
PKV_DEV uint32_t code_pair(uint32_t w) {
    if constexpr (KIND == 3) {
        const float f0 = (float)(int8_t)(w >> (HI ? 16 : 0)), f1 = (float)(int8_t)(w >> (HI ? 24 : 8));
        return __builtin_amdgcn_perm(f2u(f1), f2u(f0), 0x07060302u);
    } else {
        return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)w, 1.0f, HI));
    }
}

// 8 codes (two words) -> 8 BF16 values packed in a uint4, exactly.
template <int KIND>
PKV_DEV u32x4 codes_to_bf16(uint32_t w0, uint32_t w1) {
    return u32x4{code_pair<KIND, false>(w0), code_pair<KIND, true>(w0), code_pair<KIND, false>(w1), code_pair<KIND, true>(w1)};
}

template <bool F16>
PKV_DEV float dot2_acc(uint32_t a, uint32_t b, float c) {
    if constexpr (F16) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
    } else {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
    }
}

// V^T in LDS is [dim][64 keys], rows of 128 bytes without padding, in 8-byte groups of four keys. The second product's
// lane (row, h) multiplies, in its step over keys 16 g .. 16 g + 15, the groups 4 g + h and 4 g + 2 + h (the keys whose
// probabilities the first product left in that lane), so a row keeps those two side by side in one 16-byte slot, slot
// 2 g + h, and the operand is ONE 16-byte read. Slots are swizzled by the row, slot ^ (row & 7) ^ ((row >> 3) & 7): the
// operand reads (16 lanes: 16 adjacent rows, 16 bytes a lane) spread evenly over the banks, the stores (16 lanes: 16
// dim chunks of 8 rows, one row of each, 8 bytes a lane) two to a bank (rows 64 apart meet; a store is a small share
// of the traffic, and swapping the halves of a slot in the upper rows instead would cost the reads a register
// shuffle). Every term is a XOR of bit fields, so an address is one per-thread value XOR a compile-time constant plus
// a compile-time offset. v_place: the byte offset of key group kg in row `row`.
PKV_DEV int v_place(int kg, int row) {
    const int slot = (2 * (kg >> 2) + (kg & 1)) ^ (row & 7) ^ ((row >> 3) & 7);
    return 128 * row + 16 * slot + 8 * ((kg >> 1) & 1);
}

// Workgroups start in grid order, and a launch's tail is as long as the last ones to start: the chunks are taken
// longest first (most keys to walk; ties by index). Every wavefront ranks the chunks for itself, lane i holding chunk
// i: launches of up to 64 chunks, larger ones keep the caller's order.
PKV_DEV int chunk_by_rank(const PrefillArgs& a, int rank, int lane) {
    if (a.chunks > 64 || a.chunks < 2) return rank;
    int len = -1;
    if (lane < a.chunks) {
        const int count = a.counts ? min(a.counts[lane], a.max_count) : a.max_count;
        int64_t pos = a.positions[lane];
        pos = pos < 0 ? 0 : (pos > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : pos);
        len = (int)pos + (count > 0 ? count : 0);
    }
    int ahead = 0;      // chunks that go before this lane's
    for (int j = 0; j < a.chunks; ++j) {
        const int other = __shfl(len, j);
        ahead += (other > len || (other == len && j < lane)) ? 1 : 0;
    }
    const unsigned long long hit = __ballot(lane < a.chunks && ahead == rank);
    return __ffsll(hit) - 1;
}

}   // namespace pkv
