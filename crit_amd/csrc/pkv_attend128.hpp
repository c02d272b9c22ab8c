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

template <int KIND, bool F16, int QR, bool FUSED, bool PAGE16>
__global__ __launch_bounds__(256) void attend128_kernel(AttendArgs a) {
    constexpr int D = 128;
    constexpr int RB = (QR + 3) / 4;            // blocks of four query rows
    constexpr int EB = KIND == 0 ? 2 : 1;
    constexpr int EPT = (QR * D + 255) / 256;
    __shared__ __align__(16) float s_acc[4][QR][D];
    __shared__ float s_m[4][QR], s_l[4][QR];
    __shared__ __align__(16) uint16_t s_p[4][4][RB * 4][4];   // [wavefront][DPP row][query row][position of the row]
    __shared__ __align__(16) float s_alpha[4][4][RB * 4];
    __shared__ __align__(16) float s_rm[4][4][RB * 4], s_rl[4][4][RB * 4];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rho = lane >> 4, lam = lane & 15;
    const int b3 = (lane >> 3) & 1, b2 = (lane >> 2) & 1, b1 = (lane >> 1) & 1, b0 = lane & 1;
    const int g8 = lane >> 3, li8 = lane & 7;
    const int q4 = 2 * b2 + b3;                 // which of the DPP row's four positions this lane's score is of
    int bx = blockIdx.x;
    const int tile = bx % a.tiles;
    bx /= a.tiles;
    const int kvh = bx % a.hkv;
    const int r = bx / a.hkv;
    const int b = blockIdx.y;
    int count = a.columns;
    if (a.counts) count = min(a.counts[r], a.columns);
    const int j0 = tile * QR;
    if (j0 >= count * a.g) return;
    const int64_t first64 = a.firsts[r];
    const int c_lo = j0 / a.g;
    const int c_hi = min(count, (j0 + QR - 1) / a.g + 1);
    int64_t nk64 = first64 + c_hi;
    nk64 = nk64 < 0 ? 0 : (nk64 > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : nk64);
    const int n_keys = (int)nk64;
    const int first = (int)(first64 < 0 ? 0 : (first64 > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : first64));
    const int n_pieces = (n_keys + a.piece - 1) / a.piece;
    if (!FUSED && b >= n_pieces) return;
    const int64_t trow = (int64_t)a.rows[r] * a.tab_stride;
    const int start = a.starts[r];

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
    // The query row of this lane's score in each block, and the last position it sees.
    int my_lim[RB];
#pragma unroll
    for (int blk = 0; blk < RB; ++blk) {
        const int j = j0 + 4 * blk + 2 * b1 + b0;
        const int c = j / a.g;
        my_lim[blk] = (4 * blk + 2 * b1 + b0 < QR && c < count) ? first + c : -1;
    }
    float k_mult = a.k_mult, v_mult = a.v_mult;
    if (KIND == 1 && a.hm) k_mult = a.hm[kvh], v_mult = a.hm[a.hkv + kvh];
    const float sscale = a.sscale * (KIND == 1 ? k_mult : 1.0f);
    if (KIND != 1) v_mult = 1.0f;
    const int win = a.sliding;

    const int64_t slot_bytes = (int64_t)a.hkv * D * EB;
    const uint8_t* kbase = a.kp + (int64_t)kvh * D * EB + li8 * 16;
    const uint8_t* vbase = a.vp + (int64_t)kvh * D * EB + lam * (8 * EB);

    // Offsets of the positions this lane reads within a step: its two K rows, its row's four V rows, its score.
    const int koff[2] = {g8, 8 + g8};
    const int soff = 8 * b2 + 2 * rho + b3;

    struct Tab {
        int k[2], v[4], s;      // page table entries (PAGE16: one entry serves the step, in k[0])
    };
    auto clampn = [&](int n) { return n < n_keys ? n : n_keys - 1; };
    auto entry = [&](int n) -> int {
        int pidx = a.page_shift >= 0 ? (n >> a.page_shift) : (n / a.page);
        pidx = pidx < a.tab_width ? pidx : a.tab_width - 1;
        return a.tables[trow + pidx];
    };
    auto fetch_tab = [&](int base, Tab& t) {
        if constexpr (PAGE16) {
            t.k[0] = entry(base);      // the step's 16 positions share a page (page is a multiple of 16)
        } else {
            t.k[0] = entry(clampn(base + koff[0])), t.k[1] = entry(clampn(base + koff[1]));
#pragma unroll
            for (int kv = 0; kv < 4; ++kv) t.v[kv] = entry(clampn(base + 8 * (kv >> 1) + 2 * rho + (kv & 1)));
            if constexpr (KIND >= 2) t.s = entry(clampn(base + soff));
        }
    };
    auto slot_of = [&](int base, int off, int page_entry) -> int64_t {
        const int n = clampn(base + off);
        int in_page;
        if constexpr (PAGE16) {
            const int pidx = a.page_shift >= 0 ? (base >> a.page_shift) : (base / a.page);
            in_page = n - pidx * a.page;
        } else {
            in_page = a.page_shift >= 0 ? (n & (a.page - 1)) : (n % a.page);
        }
        return (int64_t)page_entry * a.page + in_page;
    };
    auto fetch_kv = [&](int base, const Tab& t, Step128<KIND>& buf) {
#pragma unroll
        for (int pr = 0; pr < 2; ++pr) {
            const uint8_t* row = kbase + slot_of(base, koff[pr], PAGE16 ? t.k[0] : t.k[pr]) * slot_bytes;
            if constexpr (KIND == 0) {
                buf.k[2 * pr] = *reinterpret_cast<const uint4*>(row);
                buf.k[2 * pr + 1] = *reinterpret_cast<const uint4*>(row + 128);
            } else {
                buf.k[pr] = *reinterpret_cast<const uint4*>(row);
            }
        }
#pragma unroll
        for (int kv = 0; kv < 4; ++kv) {
            const int64_t slot = slot_of(base, 8 * (kv >> 1) + 2 * rho + (kv & 1), PAGE16 ? t.k[0] : t.v[kv]);
            buf.v[kv] = *reinterpret_cast<const typename Step128<KIND>::VVec*>(vbase + slot * slot_bytes);
        }
        if constexpr (KIND >= 2) {
            const int64_t slot = slot_of(base, soff, PAGE16 ? t.k[0] : t.s);
            buf.ks = a.ks[slot * a.hkv + kvh];
            buf.vs = a.vs[slot * a.hkv + kvh];
        }
    };

    float run_m[EPT], run_l[EPT], run_a[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) run_m[e] = -INFINITY, run_l[e] = 0.0f, run_a[e] = 0.0f;

    const int part_lo = FUSED ? 0 : b;
    const int part_hi = FUSED ? min(a.parts, n_pieces) : b + 1;
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

        int pi = part, st = wave;
        if (win > 0) {
            const int wlo = first + c_lo - win + 1;
            const int below = (wlo > 0 ? wlo : 0) / a.piece - part;
            if (below > 0) pi = part + (below + a.parts - 1) / a.parts * a.parts;
        }
        auto base_of = [&]() -> int {
            if (st * 16 >= a.piece) return -1;
            const int64_t base = (int64_t)pi * a.piece + st * 16;
            return base < n_keys ? (int)base : -1;
        };
        auto advance = [&]() -> int {
            st += 4;
            if (st * 16 >= a.piece) pi += a.parts, st = wave;
            return base_of();
        };

        auto compute = [&](int base, const Step128<KIND>& buf) {
            // -- scores: each lane's partial dots of its K slices with every query row, pairs A and B
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
            // -- per block of four query rows: transposing reduction over the 8 lanes of a K row, then the softmax
            //    update of the one score the lane is left with
            float alpha_any = 1.0f;
#pragma unroll
            for (int blk = 0; blk < RB; ++blk) {
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
            // -- probabilities back, as pairs of adjacent positions per query row
            uint32_t pp[RB * 4][2];
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
            // -- P.V: pairs of positions (0,1) and (2,3) of the row against the matching pairs of V values
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

        // Three-stage software pipeline: table entries two steps ahead, K/V one step ahead, compute.
        Step128<KIND> bufA, bufB;
        Tab tabA, tabB;
        int base0 = base_of();
        if (base0 >= 0) fetch_tab(base0, tabA);
        int base1 = base0 >= 0 ? advance() : -1;
        if (base0 >= 0) fetch_kv(base0, tabA, bufA);
        if (base1 >= 0) fetch_tab(base1, tabB);
        while (base0 >= 0) {
            int base2 = base1 >= 0 ? advance() : -1;
            if (base1 >= 0) fetch_kv(base1, tabB, bufB);
            if (base2 >= 0) fetch_tab(base2, tabA);
            compute(base0, bufA);
            if (base1 < 0) break;
            base0 = base2 >= 0 ? advance() : -1;
            if (base2 >= 0) fetch_kv(base2, tabA, bufA);
            if (base0 >= 0) fetch_tab(base0, tabB);
            compute(base1, bufB);
            base1 = base0;
            base0 = base2;
        }

        // Fold the wavefront's four DPP rows: every lane needs each query row's maximum and sum of every DPP row.
#pragma unroll
        for (int blk = 0; blk < RB; ++blk) {
            if (q4 == 0) s_rm[wave][rho][4 * blk + 2 * b1 + b0] = m[blk], s_rl[wave][rho][4 * blk + 2 * b1 + b0] = l[blk];
        }
        __builtin_amdgcn_wave_barrier();
        float wm[QR], wl[QR];
#pragma unroll
        for (int rr = 0; rr < QR; ++rr) {
            float top = s_rm[wave][0][rr];
#pragma unroll
            for (int o = 1; o < 4; ++o) top = __builtin_fmaxf(top, s_rm[wave][o][rr]);
            const float sub = top == -INFINITY ? 0.0f : top;
            float lsum = 0.0f;
#pragma unroll
            for (int o = 0; o < 4; ++o) lsum = __builtin_fmaf(s_rl[wave][o][rr], exp2_fast(s_rm[wave][o][rr] - sub), lsum);
            const float w = exp2_fast(s_rm[wave][rho][rr] - sub);
#pragma unroll
            for (int d = 0; d < 8; ++d) {
                float x = acc[rr][d] * w;
                x += __shfl_xor(x, 16);
                x += __shfl_xor(x, 32);
                acc[rr][d] = x;
            }
            wm[rr] = top, wl[rr] = lsum;
        }
        if (FUSED) __syncthreads();      // the previous partition's fold has read the LDS
        if (rho == 0) {
#pragma unroll
            for (int rr = 0; rr < QR; ++rr) {
                *reinterpret_cast<float4*>(&s_acc[wave][rr][lam * 8]) = make_float4(acc[rr][0], acc[rr][1], acc[rr][2], acc[rr][3]);
                *reinterpret_cast<float4*>(&s_acc[wave][rr][lam * 8 + 4]) = make_float4(acc[rr][4], acc[rr][5], acc[rr][6], acc[rr][7]);
                if (lam == 0) s_m[wave][rr] = wm[rr], s_l[wave][rr] = wl[rr];
            }
        }
        __syncthreads();
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
                A *= v_mult;
                const int j = j0 + rr;
                const int c = j / a.g;
                if (c < count) {
                    if constexpr (FUSED) {
                        const int held = min(a.parts, (first + c + a.piece) / a.piece);
                        if (part < held) {
                            const Fold f = fold(run_m[e], run_l[e], M, L);
                            run_a[e] = __builtin_fmaf(run_a[e], f.keep, A * f.take);
                            run_m[e] = f.m, run_l[e] = f.l;
                        }
                    } else {
                        const int64_t prow = a.offsets ? (int64_t)(a.offsets[r] - a.offsets[0]) : (int64_t)r * a.columns;
                        const int64_t at = ((prow + c) * a.hq + kvh * a.g + j % a.g) * a.parts + b;
                        a.po[at * D + d] = A;
                        if (d == 0) a.pm[at] = M, a.pl[at] = L;
                    }
                }
            }
        }
    }
    if constexpr (FUSED) {
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            const int idx = tid + e * 256;
            if (idx < QR * D) {
                const int rr = idx / D, d = idx % D;
                const int j = j0 + rr;
                const int c = j / a.g;
                if (c < count) {
                    const int head = kvh * a.g + j % a.g;
                    float M = run_m[e], L = run_l[e], A = run_a[e];
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

}   // namespace pkv
