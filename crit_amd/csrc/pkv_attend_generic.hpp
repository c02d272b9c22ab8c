// Paged decode / verify-window attention, generic head widths (16 to 256, keys and values of different widths too):
// the first, plain form of the split launch, kept for what the 128-wide kernel does not cover.
//
// Work unit: one workgroup of 4 wavefronts per (row, KV head, query tile, partition). A query tile is QR rows of the
// flattened (column, query head of the KV head's group) list, so the group's heads share every K/V row read.
// Inside a wavefront LPR = max(key width, value width) / 8 lanes hold one K (or V) row, 16 bytes each (8 bytes for
// 8-bit pages), so one load instruction fetches 64/LPR whole rows; a step is four such loads for K and four for V.
// Where one of the two is narrower, the group's lanes past its width read its last 8 elements again and count for
// nothing (their query slice is zero; the outputs they accumulate are not stored). Each lane group keeps
// its own online-softmax state over the positions it reads; the groups and the four wavefronts are folded at the
// end in a fixed order, then the partition's state goes to the partials (or, fused, into the running state).
//
// SPARSE: block lists. A tile then holds rows of ONE column (the launcher picks QR dividing the group), whose list of
// block ids is copied to LDS; the positions read are the run u = 0 .. blocks_k * block_size - 1 of the list, position
// n(u) = blocks[u / block_size] * block_size + u % block_size, cut into pieces and partitions like an ordinary row's
// positions; an id of -1, a position past the column's own or past the page tables is masked. Only listed blocks are
// read. (Not fused, no sliding window: the launcher refuses those.)
//
// A column's bits depend on its own query, its own keys, `piece`, `partitions` and the page kind only: position n is
// always read by the same wavefront, lane group and step whatever the launch, masked positions contribute exact
// zeros, and every sum is an explicit FMA chain in a fixed order (built with -ffp-contract=off).
#pragma once
#include "pkv_attend_args.hpp"

namespace pkv {

struct NoFreshRows {};
struct FreshRows {
    uint4 k[4], v[4];      // the lane's 8 elements of the four positions' fresh rows, 16-bit
};
template <int KIND, bool FRESH = false>
struct StepBuf {
    using Vec = typename std::conditional<KIND == 0, uint4, uint2>::type;
    Vec k[4], v[4];
    float ks[4], vs[4];
    int pos[4];      // SPARSE: the position each of the lane group's four rows holds, -1 for none
    typename std::conditional<FRESH, FreshRows, NoFreshRows>::type f;
};


// FRESH: positions from the row's first fresh one on are read from 16-bit rows given beside the pages (row = position -
// the row's shift), unscaled: a score times the softmax scale only, a probability times 1 (_kernels.py:272-274, 291-345).
// A lane holds the same 8 elements of a row either way (16 bytes of a fresh row, 8 or 16 of a page's), so both rows are
// loaded for every position and the position picks one.
//
// DERIVE: the pool holds value rows only and a position's key is derived from its value row on read
// (paged_kv_attention/__init__.py:52-58 of the reference): k = rope(rms_norm(r) * weight, position), r the row as stored
// (codes times their scale or multiplier), rms_norm(r) = r / sqrt(mean(r * r) + eps), the "half" rotation over the
// first rotary_dim values (value i with value i + rotary_dim / 2) at the angle fp32(position) * freqs[i], all in FP32;
// the scores are FP32 products of the queries with these keys (the reference multiplies the FP32 key as two parts in
// the queries' type: the same value to about 2^-16). rotary_dim is any even width up to the head's: where it is a
// multiple of 16 a half is whole lanes and a lane's partner elements sit in one other lane.
//
// IQK (INT8 pages): each query row becomes INT8 codes at its own scale (amax / 127, at least 1e-30, rounded half away
// from zero: _kernels.py:637-643 of the reference, its int8_qk), and a page position's score is the exact integer
// product of the two rows' codes (sums below 2^24, so FP32 holds them) times both scales; a fresh position's score
// keeps the queries' 16 bits. What a prompt chunk read as window rows asks for where the matrix-core prompt kernel
// is not built for the head width.
template <int KIND, bool F16, int LPR, int QR, bool FUSED, bool SPARSE = false, bool FRESH = false, bool DERIVE = false,
          bool IQK = false>
__global__ __launch_bounds__(256) void attend_generic_kernel(AttendArgs a) {
    static_assert(!IQK || (KIND == 3 && !DERIVE && !SPARSE), "integer scores: INT8 pages, windows without lists");
    static_assert(!(SPARSE && FUSED), "block lists are read by the split launch");
    static_assert(!(SPARSE && FRESH), "block lists read the pages only");
    static_assert(!(DERIVE && SPARSE), "derived keys: windows without block lists");
    constexpr int D = LPR * 8;         // the wider of the key and value rows
    constexpr int PPI = 64 / LPR;      // positions one load instruction of a wavefront covers
    constexpr int SP = 4 * PPI;        // positions a wavefront's step covers
    constexpr int EB = KIND == 0 ? 2 : 1;
    constexpr int EPT = (QR * D + 255) / 256;   // output elements a thread folds
    __shared__ __align__(16) float s_acc[4][QR][D];
    __shared__ float s_m[4][QR], s_l[4][QR];
    __shared__ int s_blocks[SPARSE ? kMaxListedBlocks : 1];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lg = lane / LPR, li = lane % LPR;
    const int dk = a.dk, dv = a.dv;                     // the rows' own widths (multiples of 8, D the wider)
    const int lik = min(li * 8, dk - 8), liv = min(li * 8, dv - 8);      // the lane's first element of a K row and of a V row
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
    nk64 = nk64 < 0 ? 0 : (nk64 > (int64_t)a.max_keys ? (int64_t)a.max_keys : nk64);
    const int n_keys = (int)nk64;
    const int first = (int)(first64 < 0 ? 0 : (first64 > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : first64));
    const int n_run = SPARSE ? a.listed_keys : n_keys;      // the positions the partitions divide among them
    const int n_pieces = (n_run + a.piece - 1) / a.piece;
    if (!FUSED && b >= n_pieces) return;
    const int64_t trow = (int64_t)a.rows[(int64_t)r * a.rows_step] * a.tab_stride;
    const int start = a.starts[r];
    int f_first = 0x7fffffff;
    int64_t f_shift = 0;
    if constexpr (FRESH) {
        const int64_t ff = a.f_firsts[(int64_t)r * a.f_per_row];
        f_first = (int)(ff < 0 ? 0 : (ff > (int64_t)0x7fffffff ? (int64_t)0x7fffffff : ff));
        f_shift = a.f_shifts[(int64_t)r * a.f_per_row];
    }
    if constexpr (SPARSE) {      // the tile's column's list (QR divides the group: one column a tile)
        const int32_t* list = a.blocks + (int64_t)(start + c_lo) * a.blocks_stride;
        for (int i = tid; i < a.blocks_k; i += 256) s_blocks[i] = list[i];
        __syncthreads();
    }
    // SPARSE: the position behind place u of the list's run, -1 for none.
    auto listed = [&](int u) __attribute__((always_inline)) -> int {
        if (u >= a.listed_keys) return -1;
        const int e = (int)div32(a.block_div, (uint32_t)u);
        const int id = s_blocks[e];
        const int64_t n = (int64_t)id * a.block_size + (u - e * a.block_size);
        return (id >= 0 && n < n_keys) ? (int)n : -1;
    };

    // The tile's rows: column, query head, last visible position.
    int lim[QR];
    bool live[QR];
    int qhead[QR], col[QR];
#pragma unroll
    for (int rr = 0; rr < QR; ++rr) {
        const int j = j0 + rr;
        col[rr] = j / a.g;
        qhead[rr] = kvh * a.g + j % a.g;
        live[rr] = col[rr] < count;
        lim[rr] = first + col[rr];
    }
    // With a draft tree the window positions a row sees are those of its ancestors and itself.
    const bool tree = a.parents != nullptr || a.parents64 != nullptr;
    unsigned long long anc[QR];
#pragma unroll
    for (int rr = 0; rr < QR; ++rr) anc[rr] = (tree && live[rr]) ? ancestors(a, start, col[rr]) : 0ull;
    // The lane's slice of each query row: packed 16-bit pairs for 16-bit pages, FP32 for 8-bit pages.
    uint32_t qp[QR][4];
    float qf[(KIND == 0 && !DERIVE) ? 1 : QR][8];
#pragma unroll
    for (int rr = 0; rr < QR; ++rr) {
        uint4 w = make_uint4(0, 0, 0, 0);
        if (live[rr] && li * 8 < dk) {
            w = *reinterpret_cast<const uint4*>(a.q + ((int64_t)(start + col[rr]) * a.q_st + (int64_t)qhead[rr] * a.q_sh + li * 8) * 2);
        }
        qp[rr][0] = w.x, qp[rr][1] = w.y, qp[rr][2] = w.z, qp[rr][3] = w.w;
        if constexpr (KIND != 0 || DERIVE) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                qf[rr][2 * j] = F16 ? f16_lo(qp[rr][j]) : bf16_lo(qp[rr][j]);
                qf[rr][2 * j + 1] = F16 ? f16_hi(qp[rr][j]) : bf16_hi(qp[rr][j]);
            }
        }
    }
    float qi[IQK ? QR : 1][8], q_scale[IQK ? QR : 1];      // IQK: the rows' codes (as FP32 integers) and scales
    if constexpr (IQK) {
#pragma unroll
        for (int rr = 0; rr < QR; ++rr) {
            float amax = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j) amax = __builtin_fmaxf(amax, __builtin_fabsf(qf[rr][j]));
            amax = group_max<LPR>(amax);
            q_scale[rr] = __builtin_fmaxf(__fdiv_rn(amax, 127.0f), 1e-30f);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float f = __fdiv_rn(qf[rr][j], q_scale[rr]);
                qi[rr][j] = (float)(int)(f >= 0.0f ? f + 0.5f : f - 0.5f);      // (a NaN row gives codes of 0, as the cast does)
            }
        }
    }
    float k_mult = a.k_mult, v_mult = a.v_mult;
    if (KIND == 1 && a.hm) k_mult = a.hm[kvh], v_mult = a.hm[a.hkv + kvh];
    const float sscale = a.sscale * (KIND == 1 ? k_mult : 1.0f);
    if (KIND != 1) v_mult = 1.0f;
    const int win = a.sliding;

    const uint8_t* kbase = a.kp + ((int64_t)kvh * dk + lik) * EB;
    const uint8_t* vbase = a.vp + ((int64_t)kvh * dv + liv) * EB;
    const int64_t slot_bytes_k = (int64_t)a.hkv * dk * EB, slot_bytes_v = (int64_t)a.hkv * dv * EB;

    auto fetch_tab = [&](int base, int (&tab)[4], int (&pos)[4]) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            int n = base + k * PPI + lg;
            if constexpr (SPARSE) {
                pos[k] = listed(n);
                n = pos[k] >= 0 ? pos[k] : 0;      // (a masked place reads position 0: any valid address)
            } else {
                n = n < n_keys ? n : n_keys - 1;
            }
            int pidx = a.page_shift >= 0 ? (n >> a.page_shift) : (n / a.page);
            pidx = pidx < a.tab_width ? pidx : a.tab_width - 1;
            tab[k] = a.tables[trow + pidx];
        }
    };
    auto fetch_kv = [&](int base, const int (&tab)[4], const int (&pos)[4], StepBuf<KIND, FRESH>& buf) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            int n = base + k * PPI + lg;
            if constexpr (SPARSE) {
                buf.pos[k] = pos[k];
                n = pos[k] >= 0 ? pos[k] : 0;
            } else {
                n = n < n_keys ? n : n_keys - 1;
            }
            const int in_page = a.page_shift >= 0 ? (n & (a.page - 1)) : (n % a.page);
            const int64_t slot = (int64_t)tab[k] * a.page + in_page;
            if constexpr (!DERIVE) buf.k[k] = *reinterpret_cast<const typename StepBuf<KIND>::Vec*>(kbase + slot * slot_bytes_k);
            if constexpr (KIND == 0) buf.v[k] = load_once16(vbase + slot * slot_bytes_v);
            else buf.v[k] = load_once8(vbase + slot * slot_bytes_v);
            if constexpr (KIND >= 2) {
                if constexpr (!DERIVE) buf.ks[k] = a.ks[slot * a.hkv + kvh];
                buf.vs[k] = a.vs[slot * a.hkv + kvh];
            }
            if constexpr (FRESH) {      // (unconditional too: a position below the first fresh one reads row 0 or its own clamped)
                int64_t row = (int64_t)n - f_shift;
                row = row < 0 ? 0 : (row >= a.f_rows ? a.f_rows - 1 : row);
                if constexpr (!DERIVE) buf.f.k[k] = *reinterpret_cast<const uint4*>(a.fk + (row * a.f_stride_k + (int64_t)kvh * dk + lik) * 2);
                buf.f.v[k] = load_once16(a.fv + (row * a.f_stride_v + (int64_t)kvh * dv + liv) * 2);
            }
        }
    };

    // Running state of the fused fold (one per output element of this thread).
    float run_m[EPT], run_l[EPT], run_a[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) run_m[e] = -INFINITY, run_l[e] = 0.0f, run_a[e] = 0.0f;

    const int part_lo = FUSED ? 0 : b;
    const int part_hi = FUSED ? min(a.parts, n_pieces) : b + 1;
    for (int part = part_lo; part < part_hi; ++part) {
        float m[QR], l[QR], acc[QR][8];
#pragma unroll
        for (int rr = 0; rr < QR; ++rr) {
            m[rr] = -INFINITY, l[rr] = 0.0f;
#pragma unroll
            for (int d = 0; d < 8; ++d) acc[rr][d] = 0.0f;
        }
        // This wavefront's steps: steps wave, wave + 4, ... of pieces part, part + parts, ...
        int pi = part, st = wave;
        if (win > 0) {   // pieces wholly below the tile's window are skipped (no row sees them)
            const int wlo = first + c_lo - win + 1;
            const int below = (wlo > 0 ? wlo : 0) / a.piece - part;
            if (below > 0) pi = part + (below + a.parts - 1) / a.parts * a.parts;
        }
        auto base_of = [&]() __attribute__((always_inline)) -> int {
            if (st * SP >= a.piece) return -1;
            const int64_t base = (int64_t)pi * a.piece + st * SP;
            return base < n_run ? (int)base : -1;
        };
        auto advance = [&]() __attribute__((always_inline)) -> int {
            st += 4;
            if (st * SP >= a.piece) pi += a.parts, st = wave;
            return base_of();
        };

        // The lane's 8 values of position k's value row as the page holds them (codes, not yet times their scale).
        auto stored_values = [&](const StepBuf<KIND, FRESH>& buf, int k, float (&vf)[8]) __attribute__((always_inline)) {
            if constexpr (KIND == 0) {
                const uint32_t vw[4] = {buf.v[k].x, buf.v[k].y, buf.v[k].z, buf.v[k].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    vf[2 * j] = F16 ? f16_lo(vw[j]) : bf16_lo(vw[j]);
                    vf[2 * j + 1] = F16 ? f16_hi(vw[j]) : bf16_hi(vw[j]);
                }
            } else if constexpr (KIND == 3) {
                const uint32_t w2[2] = {buf.v[k].x, buf.v[k].y};
#pragma unroll
                for (int j = 0; j < 8; ++j) vf[j] = (float)(int8_t)(w2[j / 4] >> (8 * (j % 4)));
            } else {
                const f32x2 a0 = e4m3_pair<false>(buf.v[k].x), a1 = e4m3_pair<true>(buf.v[k].x);
                const f32x2 a2 = e4m3_pair<false>(buf.v[k].y), a3 = e4m3_pair<true>(buf.v[k].y);
                vf[0] = a0.x, vf[1] = a0.y, vf[2] = a1.x, vf[3] = a1.y;
                vf[4] = a2.x, vf[5] = a2.y, vf[6] = a3.x, vf[7] = a3.y;
            }
        };
        // DERIVE: position n's key from its value row (a fresh position's from its fresh value row, as it is given).
        auto derived_key = [&](const StepBuf<KIND, FRESH>& buf, int k, int n, bool is_fresh, float (&kf)[8]) __attribute__((always_inline)) {
            stored_values(buf, k, kf);
            const float rs = KIND >= 2 ? buf.vs[k] : (KIND == 1 ? v_mult : 1.0f);
#pragma unroll
            for (int j = 0; j < 8; ++j) kf[j] *= rs;
            if constexpr (FRESH) {
                const uint32_t fw[4] = {buf.f.v[k].x, buf.f.v[k].y, buf.f.v[k].z, buf.f.v[k].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    kf[2 * j] = is_fresh ? (F16 ? f16_lo(fw[j]) : bf16_lo(fw[j])) : kf[2 * j];
                    kf[2 * j + 1] = is_fresh ? (F16 ? f16_hi(fw[j]) : bf16_hi(fw[j])) : kf[2 * j + 1];
                }
            }
            float ss = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j) ss = __builtin_fmaf(kf[j], kf[j], ss);
            ss = group_sum<LPR>(ss);
            const float rn = 1.0f / __builtin_sqrtf(ss / (float)D + a.derive_eps);
            const float* weight = a.derive_table + (a.derive_rot >> 1);
#pragma unroll
            for (int j = 0; j < 8; ++j) kf[j] = kf[j] * rn * (a.derive_weighted ? weight[li * 8 + j] : 1.0f);
            // Element e = 8 li + j turns with element e + h (e below h = rotary_dim / 2) or e - h (h <= e < rotary_dim).
            const int h = a.derive_rot >> 1, hl = h >> 3, hs = h & 7;      // the partner: hl lanes and hs places away
            float other[8];
            if (hs == 0) {      // halves of whole lanes: the partner sits at the same place of the lane hl away
                const bool low = li < hl, turns = li < 2 * hl;
                const int from = turns ? (low ? lane + hl : lane - hl) : lane;
#pragma unroll
                for (int j = 0; j < 8; ++j) other[j] = __shfl(kf[j], from);
            } else {
                // Any even width: place s of a lane is the partner of place (s - hs) mod 8 of the lower half's elements
                // (in the lane hl, or hl + 1, below) and of place (s + hs) mod 8 of the upper half's (hl, or hl + 1,
                // above); both places are the same for every lane, so each is one shuffle and a select.
#pragma unroll
                for (int j = 0; j < 8; ++j) other[j] = 0.0f;
#pragma unroll
                for (int s = 0; s < 8; ++s) {
                    const int jl = (s - hs) & 7, ju = (s + hs) & 7;
                    const float up = __shfl(kf[s], lane + hl + (jl + hs >= 8 ? 1 : 0));       // for an element of the lower half
                    const float down = __shfl(kf[s], lane - hl - (ju < hs ? 1 : 0));          // for one of the upper half
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const int e = li * 8 + j;
                        other[j] = (j == jl && e < h) ? up : ((j == ju && e >= h && e < a.derive_rot) ? down : other[j]);
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int e = li * 8 + j;
                const bool low = e < h, turns = e < a.derive_rot;
                float sn, cs;
                sincosf((float)n * a.derive_table[turns ? (low ? e : e - h) : 0], &sn, &cs);
                const float turned = low ? kf[j] * cs - other[j] * sn : kf[j] * cs + other[j] * sn;
                kf[j] = turns ? turned : kf[j];
            }
        };

        auto compute = [&](int base, const StepBuf<KIND, FRESH>& buf) __attribute__((always_inline)) {
            float s[4][QR];
            bool isf[4];      // FRESH: the position's row is a fresh one
#pragma unroll
            for (int k = 0; k < 4; ++k) isf[k] = FRESH && base + k * PPI + lg >= f_first;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                uint32_t kw[4];
                float kf[8];
                if constexpr (DERIVE) {
                    const int n = base + k * PPI + lg;
                    derived_key(buf, k, n < n_keys ? n : n_keys - 1, isf[k], kf);
                } else if constexpr (KIND == 0) {
                    kw[0] = buf.k[k].x, kw[1] = buf.k[k].y, kw[2] = buf.k[k].z, kw[3] = buf.k[k].w;
                } else if constexpr (KIND == 3) {
                    const uint32_t w2[2] = {buf.k[k].x, buf.k[k].y};
#pragma unroll
                    for (int j = 0; j < 8; ++j) kf[j] = (float)(int8_t)(w2[j / 4] >> (8 * (j % 4)));
                } else {
                    const f32x2 a0 = e4m3_pair<false>(buf.k[k].x), a1 = e4m3_pair<true>(buf.k[k].x);
                    const f32x2 a2 = e4m3_pair<false>(buf.k[k].y), a3 = e4m3_pair<true>(buf.k[k].y);
                    kf[0] = a0.x, kf[1] = a0.y, kf[2] = a1.x, kf[3] = a1.y;
                    kf[4] = a2.x, kf[5] = a2.y, kf[6] = a3.x, kf[7] = a3.y;
                }
                if constexpr (FRESH && !DERIVE) {
                    const uint32_t fw[4] = {buf.f.k[k].x, buf.f.k[k].y, buf.f.k[k].z, buf.f.k[k].w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if constexpr (KIND == 0) {
                            kw[j] = isf[k] ? fw[j] : kw[j];
                        } else {
                            kf[2 * j] = isf[k] ? (F16 ? f16_lo(fw[j]) : bf16_lo(fw[j])) : kf[2 * j];
                            kf[2 * j + 1] = isf[k] ? (F16 ? f16_hi(fw[j]) : bf16_hi(fw[j])) : kf[2 * j + 1];
                        }
                    }
                }
#pragma unroll
                for (int rr = 0; rr < QR; ++rr) {
                    float d = 0.0f;
                    if constexpr (KIND == 0 && !DERIVE) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            if constexpr (F16) {
                                d = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, qp[rr][j]), __builtin_bit_cast(f16x2, kw[j]), d, false);
                            } else {
                                d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, qp[rr][j]), __builtin_bit_cast(bf16x2, kw[j]), d, false);
                            }
                        }
                    } else {
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            float qv = qf[rr][j];
                            if constexpr (IQK) qv = (FRESH && isf[k]) ? qv : qi[rr][j];
                            d = __builtin_fmaf(qv, kf[j], d);
                        }
                    }
                    s[k][rr] = group_sum<LPR>(d);
                }
            }
            // Scale, mask, and one online-softmax update per row over the step's four positions of this lane group.
#pragma unroll
            for (int rr = 0; rr < QR; ++rr) {
                float top = -INFINITY;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int n = SPARSE ? buf.pos[k] : base + k * PPI + lg;
                    float x = s[k][rr] * ((isf[k] || DERIVE) ? a.sscale : (KIND >= 2 ? sscale * buf.ks[k] : sscale));
                    if constexpr (IQK) x = isf[k] ? x : x * q_scale[rr];
                    bool vis = n <= lim[rr] && n < n_keys;
                    if constexpr (SPARSE) vis = vis && n >= 0;
                    if (tree) vis = vis && (n < first || ((anc[rr] >> ((n - first) & 63)) & 1ull) != 0);
                    if (win > 0) vis = vis && n > lim[rr] - win;
                    x = vis ? x : -INFINITY;
                    s[k][rr] = x;
                    top = __builtin_fmaxf(top, x);
                }
                const float m_new = __builtin_fmaxf(m[rr], top);
                const float sub = m_new == -INFINITY ? 0.0f : m_new;
                const float alpha = exp2_fast(m[rr] - sub);
                float sum = 0.0f;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float p = exp2_fast(s[k][rr] - sub);
                    sum += p;
                    if constexpr (FRESH && KIND != 0) {      // (FP8 pages' one value multiplier rides here too: a fresh row counts as given)
                        s[k][rr] = isf[k] ? p : p * (KIND >= 2 ? buf.vs[k] : v_mult);
                    } else {
                        s[k][rr] = KIND >= 2 ? p * buf.vs[k] : p;
                    }
                }
                l[rr] = __builtin_fmaf(l[rr], alpha, sum);
                m[rr] = m_new;
#pragma unroll
                for (int d = 0; d < 8; ++d) acc[rr][d] *= alpha;
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                float vf[8];
                stored_values(buf, k, vf);
                if constexpr (FRESH) {
                    const uint32_t fw[4] = {buf.f.v[k].x, buf.f.v[k].y, buf.f.v[k].z, buf.f.v[k].w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        vf[2 * j] = isf[k] ? (F16 ? f16_lo(fw[j]) : bf16_lo(fw[j])) : vf[2 * j];
                        vf[2 * j + 1] = isf[k] ? (F16 ? f16_hi(fw[j]) : bf16_hi(fw[j])) : vf[2 * j + 1];
                    }
                }
#pragma unroll
                for (int rr = 0; rr < QR; ++rr) {
#pragma unroll
                    for (int d = 0; d < 8; ++d) acc[rr][d] = __builtin_fmaf(s[k][rr], vf[d], acc[rr][d]);
                }
            }
        };

        // Three-stage software pipeline: table entries two steps ahead, K/V one step ahead, compute. Every load of the
        // loop is issued unconditionally (past the wavefront's last step it re-reads its first step, which the caches
        // hold): with loads under conditions the compiler waits for all outstanding loads at every use.
        StepBuf<KIND, FRESH> bufA, bufB;
        int tabA[4], tabB[4], posA[4], posB[4];
        int base0 = base_of();
        if (base0 >= 0) {
            const int again = base0;
            auto safe = [&](int base) __attribute__((always_inline)) { return base >= 0 ? base : again; };
            fetch_tab(base0, tabA, posA);
            int base1 = advance();
            fetch_tab(safe(base1), tabB, posB);
            fetch_kv(base0, tabA, posA, bufA);
            for (;;) {
                const int base2 = base1 >= 0 ? advance() : -1;
                fetch_kv(safe(base1), tabB, posB, bufB);
                fetch_tab(safe(base2), tabA, posA);
                compute(base0, bufA);
                if (base1 < 0) break;
                const int base3 = base2 >= 0 ? advance() : -1;
                fetch_kv(safe(base2), tabA, posA, bufA);
                fetch_tab(safe(base3), tabB, posB);
                compute(base1, bufB);
                if (base2 < 0) break;
                base0 = base2, base1 = base3;
            }
        }

        // Fold the wavefront's lane groups (butterfly: every lane ends with the same bits), then the four wavefronts
        // through LDS in wavefront order.
#pragma unroll
        for (int rr = 0; rr < QR; ++rr) {
            const float top = max_over_groups<LPR>(m[rr]);
            const float sub = top == -INFINITY ? 0.0f : top;
            const float w = exp2_fast(m[rr] - sub);
            const float lw = sum_over_groups<LPR>(l[rr] * w);
#pragma unroll
            for (int d = 0; d < 8; ++d) acc[rr][d] = sum_over_groups<LPR>(acc[rr][d] * w);
            m[rr] = top, l[rr] = lw;
        }
        if (FUSED) __syncthreads();      // the previous partition's fold has read the LDS
        if (lg == 0) {
#pragma unroll
            for (int rr = 0; rr < QR; ++rr) {
                *reinterpret_cast<float4*>(&s_acc[wave][rr][li * 8]) = make_float4(acc[rr][0], acc[rr][1], acc[rr][2], acc[rr][3]);
                *reinterpret_cast<float4*>(&s_acc[wave][rr][li * 8 + 4]) = make_float4(acc[rr][4], acc[rr][5], acc[rr][6], acc[rr][7]);
                if (li == 0) s_m[wave][rr] = m[rr], s_l[wave][rr] = l[rr];
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
                if constexpr (!(FRESH && KIND == 1)) A *= v_mult;      // (with fresh rows the multiplier went in a position at a time)
                const int j = j0 + rr;
                const int c = j / a.g;
                if (c < count && d < dv) {
                    if constexpr (FUSED) {
                        // A column folds the partitions that hold its positions, as the merge does.
                        const int held = min(a.parts, (min(first + c + 1, a.max_keys) + a.piece - 1) / a.piece);
                        if (part < held) {
                            const Fold f = fold(run_m[e], run_l[e], M, L);
                            run_a[e] = __builtin_fmaf(run_a[e], f.keep, A * f.take);
                            run_m[e] = f.m, run_l[e] = f.l;
                        }
                    } else {
                        const int64_t prow = a.offsets ? (int64_t)(a.offsets[r] - a.offsets[0]) : (int64_t)r * a.columns;
                        const int64_t at = ((prow + c) * a.hq + kvh * a.g + j % a.g) * a.parts + b;
                        a.po[at * dv + d] = A;
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
                if (c < count && d < dv) {
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
