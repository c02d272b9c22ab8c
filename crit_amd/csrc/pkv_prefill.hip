// Chunked prefill over paged KV on the matrix cores (v_mfma_f32_32x32x16 bf16/f16).
//
// Work unit: one workgroup of 4 wavefronts per (query tile, KV head, chunk). A query tile is 128 rows of the
// flattened (token, query head of the KV head's group) list, 32 rows per wavefront, so a K/V block is staged once for
// the whole GQA group. Keys are walked in absolute blocks of 64 positions (block b = positions 64b .. 64b+63 whatever
// the chunk), gathered through the page table into LDS: K row-major, V transposed ([dim][key]) so both matrix
// products read their contraction index contiguously.
//
// Both products are computed transposed, S^T = K Q^T and O^T = V^T P^T: in the accumulator layout of a 32x32 MFMA a
// lane then holds ONE query row (column l % 32) and 16 keys (or 16 output dims) of it, so the online softmax is
// per-lane arithmetic plus one exchange between the two half-waves, and the probabilities a lane produced are exactly
// the B operand it must feed to the second product: no shuffle, no LDS round trip for P.
//
// A token's bits follow its own positions only: the key blocks are absolute, masked keys contribute exact zeros.
#include "pkv_common.hpp"
#include "pkv_launch.hpp"

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
    int tab_width, chunks, max_count, hq, hkv, g, page, page_shift, sliding, out_dtype;
    float sscale, k_mult, v_mult;
};

constexpr int BM = 128;   // query rows a workgroup holds
constexpr int BN = 64;    // keys a block holds

// 8 codes (two words of E4M3 or INT8) -> 8 BF16 values packed in a uint4, exactly.
template <int KIND>
PKV_DEV uint4 codes_to_bf16(uint32_t w0, uint32_t w1) {
    float f[8];
    if constexpr (KIND == 3) {
#pragma unroll
        for (int j = 0; j < 4; ++j) f[j] = (float)(int8_t)(w0 >> (8 * j)), f[4 + j] = (float)(int8_t)(w1 >> (8 * j));
    } else {
        const f32x2 a0 = e4m3_pair<false>(w0), a1 = e4m3_pair<true>(w0), a2 = e4m3_pair<false>(w1), a3 = e4m3_pair<true>(w1);
        f[0] = a0.x, f[1] = a0.y, f[2] = a1.x, f[3] = a1.y, f[4] = a2.x, f[5] = a2.y, f[6] = a3.x, f[7] = a3.y;
    }
    uint4 r;
    r.x = (f2u(f[0]) >> 16) | (f2u(f[1]) & 0xffff0000u);
    r.y = (f2u(f[2]) >> 16) | (f2u(f[3]) & 0xffff0000u);
    r.z = (f2u(f[4]) >> 16) | (f2u(f[5]) & 0xffff0000u);
    r.w = (f2u(f[6]) >> 16) | (f2u(f[7]) & 0xffff0000u);
    return r;
}

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

template <bool F16>
PKV_DEV float dot2_acc(uint32_t a, uint32_t b, float c) {
    if constexpr (F16) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
    } else {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
    }
}

// V^T in LDS is [dim][64 keys], rows of 128 bytes without padding; the 8-byte group of four keys g of row `row` sits
// at group g ^ swz(row): the stores (lanes vary the dim chunk and the key group) and the operand reads (lanes vary
// the dim and the half-wave's key group) both spread over all banks.
PKV_DEV int swz(int row) { return (row & 15) ^ ((row >> 3) & 15); }

template <int KIND, bool F16, int D>
__global__ __launch_bounds__(256, 2) void prefill_kernel(PrefillArgs a) {
    constexpr int KS = D / 16;          // k-steps of the first product
    constexpr int NB = D / 32;          // 32-wide output blocks of the second product
    constexpr int KSTR = D + 8;         // K row stride in LDS (16-bit elements): 16 bytes of padding
    constexpr int EB = KIND == 0 ? 2 : 1;
    constexpr int CH = D * EB / 16;     // 16-byte chunks of one K or V row in the pages
    constexpr int KPASS = BN * CH / 256;   // passes of 256 threads over a K block, rows contiguous over lanes
    constexpr int VGROUPS = 16 * CH;    // 16-bit pages: (group of four keys, 16-byte chunk) pairs of a V block
    constexpr int VGP = (VGROUPS + 255) / 256;
    constexpr int VPASS = KIND == 0 ? 4 * VGP : CH / 4;
    __shared__ __align__(16) uint16_t k_lds[2][BN * KSTR];
    __shared__ __align__(16) uint16_t v_lds[2][D * BN];
    __shared__ float ks_lds[2][BN], vs_lds[2][BN];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n32 = lane & 31, h = lane >> 5;
    const int tile = gridDim.x - 1 - blockIdx.x;      // later tiles see more keys: start them first
    const int kvh = blockIdx.y, z = blockIdx.z;
    int count = a.max_count;
    if (a.counts) count = min(a.counts[z], a.max_count);
    if ((int64_t)tile * BM >= (int64_t)count * a.g) return;
    const int start = a.starts ? a.starts[z] : 0;
    int64_t pos64 = a.positions[z];
    pos64 = pos64 < 0 ? 0 : (pos64 > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : pos64);
    const int pos = (int)pos64;
    const int64_t trow = (int64_t)(a.table_rows ? a.table_rows[z] : z) * a.tab_stride;

    // This lane's query row.
    const int j = tile * BM + wave * 32 + n32;
    const int t = j / a.g, head = kvh * a.g + j % a.g;
    const bool live = t < count;
    const int lim = live ? pos + t : -1;
    uint4 qreg[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        qreg[ks] = make_uint4(0, 0, 0, 0);
        if (live) {
            qreg[ks] = *reinterpret_cast<const uint4*>(a.q + ((int64_t)(start + t) * a.q_st + (int64_t)head * a.q_sh + 16 * ks + 8 * h) * 2);
        }
    }
    // The lowest limit among the wavefront's live rows: key blocks wholly at or below it need no mask.
    int wave_lo = live ? lim : 0x7fffffff;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) wave_lo = min(wave_lo, __shfl_xor(wave_lo, o));
    float k_mult = a.k_mult, v_mult = a.v_mult;
    if (KIND == 1 && a.hm) k_mult = a.hm[kvh], v_mult = a.hm[a.hkv + kvh];
    const float sscale = a.sscale * (KIND == 1 ? k_mult : 1.0f);
    if (KIND != 1) v_mult = 1.0f;
    const int win = a.sliding;

    const int t_lo = tile * BM / a.g;
    const int t_hi = min(count - 1, (tile * BM + BM - 1) / a.g);
    const int n_max = pos + count - 1;                 // the chunk's last written position
    const int kt_hi = (pos + t_hi) / BN;
    int kt_lo = 0;
    if (win > 0) kt_lo = max(0, pos + t_lo - win + 1) / BN;

    // The page table entry and the slot of a position (positions past the chunk's last written one read that one).
    // One 4-byte load whatever the table's type: an int64 entry's low word holds the page number (little endian).
    const uint8_t* tab_bytes = a.tables ? reinterpret_cast<const uint8_t*>(a.tables) : reinterpret_cast<const uint8_t*>(a.tables64);
    const int tab_shift = a.tables ? 2 : 3;
    auto entry_of = [&](int n) __attribute__((always_inline)) -> int {
        n = n < n_max ? n : n_max;
        int pidx = a.page_shift >= 0 ? (n >> a.page_shift) : (n / a.page);
        pidx = pidx < a.tab_width ? pidx : a.tab_width - 1;
        return *reinterpret_cast<const int*>(tab_bytes + ((trow + pidx) << tab_shift));
    };
    auto slot_at = [&](int n, int pg) __attribute__((always_inline)) -> int64_t {
        n = n < n_max ? n : n_max;
        const int pidx = a.page_shift >= 0 ? (n >> a.page_shift) : (n / a.page);
        return (int64_t)pg * a.page + (n - pidx * a.page);
    };
    const int64_t slot_bytes = (int64_t)a.hkv * D * EB;
    const uint8_t* kbase = a.kp + (int64_t)kvh * D * EB;
    const uint8_t* vbase = a.vp + (int64_t)kvh * D * EB;

    // Global -> registers -> LDS. K: rows contiguous over lanes. V, 16-bit pages: a thread takes one 16-byte chunk of
    // four adjacent keys and stores it transposed as eight 8-byte groups; 8-bit pages: lane = key, wavefront = chunk.
    // The page table entries of a block are fetched one block before its rows (load_entries, then load_block): a
    // row's address depends on its entry, and a wait on an entry would also wait on every row load issued before it.
    constexpr int NENT = KPASS + (KIND == 0 ? VGP * 4 : 1) + (KIND >= 2 ? 1 : 0);
    u32x4 kreg[KPASS], vreg[VPASS];
    int ent[NENT];
    float ksreg = 1.0f, vsreg = 1.0f;
    auto load_entries = [&](int kt) __attribute__((always_inline)) {
        const int n0 = kt * BN;
        static_for<KPASS>([&](auto pc) __attribute__((always_inline)) {
            constexpr int p = decltype(pc)::value;
            ent[p] = entry_of(n0 + (p * 256 + tid) / CH);
        });
        if constexpr (KIND == 0) {
            static_for<VGP * 4>([&](auto ic) __attribute__((always_inline)) {
                constexpr int i = decltype(ic)::value;
                const int kg = ((i / 4) * 256 + tid) % VGROUPS / CH;
                ent[KPASS + i] = entry_of(n0 + 4 * kg + i % 4);
            });
        } else {
            ent[KPASS] = entry_of(n0 + lane);
        }
        if constexpr (KIND >= 2) ent[NENT - 1] = entry_of(n0 + (tid & (BN - 1)));
    };
    auto load_block = [&](int kt) __attribute__((always_inline)) {
        const int n0 = kt * BN;
        static_for<KPASS>([&](auto pc) __attribute__((always_inline)) {
            constexpr int p = decltype(pc)::value;
            const int idx = p * 256 + tid;
            const int kk = idx / CH, c = idx % CH;
            kreg[p] = *reinterpret_cast<const u32x4*>(kbase + slot_at(n0 + kk, ent[p]) * slot_bytes + c * 16);
        });
        if constexpr (KIND == 0) {
            static_for<VGP * 4>([&](auto ic) __attribute__((always_inline)) {
                constexpr int i = decltype(ic)::value;
                const int idx = ((i / 4) * 256 + tid) % VGROUPS;      // D = 64: the upper half of the workgroup repeats the lower
                const int kg = idx / CH, c = idx % CH;
                vreg[i] = *reinterpret_cast<const u32x4*>(vbase + slot_at(n0 + 4 * kg + i % 4, ent[KPASS + i]) * slot_bytes + c * 16);
            });
        } else {
            const int64_t vslot = slot_at(n0 + lane, ent[KPASS]);
            static_for<VPASS>([&](auto pc) __attribute__((always_inline)) {
                constexpr int p = decltype(pc)::value;
                vreg[p] = *reinterpret_cast<const u32x4*>(vbase + vslot * slot_bytes + (4 * p + wave) * 16);
            });
        }
        if constexpr (KIND >= 2) {
            const int64_t s = slot_at(n0 + (tid & (BN - 1)), ent[NENT - 1]);
            ksreg = a.ks[s * a.hkv + kvh], vsreg = a.vs[s * a.hkv + kvh];
        }
    };
    auto store_block = [&](int buf) __attribute__((always_inline)) {
        uint16_t* kl = k_lds[buf];
        uint16_t* vl = v_lds[buf];
        static_for<KPASS>([&](auto pc) __attribute__((always_inline)) {
            constexpr int p = decltype(pc)::value;
            const int idx = p * 256 + tid;
            const int kk = idx / CH, c = idx % CH;
            if constexpr (KIND == 0) {
                *reinterpret_cast<u32x4*>(&kl[kk * KSTR + c * 8]) = kreg[p];
            } else {
                *reinterpret_cast<uint4*>(&kl[kk * KSTR + c * 16]) = codes_to_bf16<KIND>(kreg[p].x, kreg[p].y);
                *reinterpret_cast<uint4*>(&kl[kk * KSTR + c * 16 + 8]) = codes_to_bf16<KIND>(kreg[p].z, kreg[p].w);
            }
        });
        if constexpr (KIND == 0) {
            static_for<VGP>([&](auto pc) __attribute__((always_inline)) {
                constexpr int p = decltype(pc)::value;
                const int idx = (p * 256 + tid) % VGROUPS;      // repeated groups store the same bytes twice
                const int kg = idx / CH, c = idx % CH;
                const uint32_t w0[4] = {vreg[4 * p].x, vreg[4 * p].y, vreg[4 * p].z, vreg[4 * p].w};
                const uint32_t w1[4] = {vreg[4 * p + 1].x, vreg[4 * p + 1].y, vreg[4 * p + 1].z, vreg[4 * p + 1].w};
                const uint32_t w2[4] = {vreg[4 * p + 2].x, vreg[4 * p + 2].y, vreg[4 * p + 2].z, vreg[4 * p + 2].w};
                const uint32_t w3[4] = {vreg[4 * p + 3].x, vreg[4 * p + 3].y, vreg[4 * p + 3].z, vreg[4 * p + 3].w};
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int row = c * 8 + i;
                    const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
                    const uint32_t k01 = __builtin_amdgcn_perm(w1[i / 2], w0[i / 2], sel);
                    const uint32_t k23 = __builtin_amdgcn_perm(w3[i / 2], w2[i / 2], sel);
                    *reinterpret_cast<uint2*>(&vl[row * BN + 4 * (kg ^ swz(row))]) = make_uint2(k01, k23);
                }
            });
        } else {
            static_for<VPASS>([&](auto pc) __attribute__((always_inline)) {
                constexpr int p = decltype(pc)::value;
                const int c = 4 * p + wave;
                const uint4 lo = codes_to_bf16<KIND>(vreg[p].x, vreg[p].y), hi = codes_to_bf16<KIND>(vreg[p].z, vreg[p].w);
                const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
                for (int i = 0; i < 8; ++i) {
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        const int row = c * 16 + 2 * i + half;
                        vl[row * BN + 4 * ((lane >> 2) ^ swz(row)) + (lane & 3)] = (uint16_t)(half ? w[i] >> 16 : w[i] & 0xffffu);
                    }
                }
            });
        }
        if constexpr (KIND >= 2) {
            if (tid < BN) ks_lds[buf][tid] = ksreg, vs_lds[buf][tid] = vsreg;
        }
    };

    f32x16 o[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[nb][v] = 0.0f;
    float m = -INFINITY, l = 0.0f;

    // Double-buffered LDS, one barrier a block: block kt is multiplied from buffer kt & 1 while block kt + 1 (already
    // in registers) is stored into the other buffer, block kt + 2 is fetched from the pages and the table entries of
    // block kt + 3 are read. Every load of the loop is unconditional (past the last block it repeats the last one), so
    // the compiler counts the outstanding loads exactly instead of waiting for all of them.
    auto upto = [&](int kt) __attribute__((always_inline)) { return kt < kt_hi ? kt : kt_hi; };
    load_entries(kt_lo);
    load_block(kt_lo);
    load_entries(upto(kt_lo + 1));
    store_block(kt_lo & 1);
    load_block(upto(kt_lo + 1));
    load_entries(upto(kt_lo + 2));
    __syncthreads();
    for (int kt = kt_lo; kt <= kt_hi; ++kt) {
        const int buf = kt & 1;
        const uint16_t* kl = k_lds[buf];
        const uint16_t* vl = v_lds[buf];
        // S^T = K Q^T: two blocks of 32 keys x this wavefront's 32 rows.
        f32x16 s[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int v = 0; v < 16; ++v) s[kb][v] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const uint4 kop = *reinterpret_cast<const uint4*>(&kl[(32 * kb + n32) * KSTR + 16 * ks + 8 * h]);
                s[kb] = mfma<F16>(kop, qreg[ks], s[kb]);
            }
        }
        // The next block goes into the other buffer while this one is multiplied (its readers passed the barrier).
        store_block(buf ^ 1);
        load_block(upto(kt + 2));
        load_entries(upto(kt + 3));
        // Scale (and mask where the block is not wholly visible); the lane holds keys 32 kb + 8 (v / 4) + 4 h + v % 4
        // of its own row.
        const bool masked = win > 0 || kt * BN + BN - 1 > wave_lo;
        float top = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int kin = 32 * kb + 8 * (v / 4) + 4 * h + v % 4;
                float x = s[kb][v] * (KIND >= 2 ? sscale * ks_lds[buf][kin] : sscale);
                if (masked) {
                    const int n = kt * BN + kin;
                    bool vis = n <= lim;
                    if (win > 0) vis = vis && n > lim - win;
                    x = vis ? x : -INFINITY;
                }
                s[kb][v] = x;
                top = __builtin_fmaxf(top, x);
            }
        }
        top = __builtin_fmaxf(top, __shfl_xor(top, 32));
        const float m_new = __builtin_fmaxf(m, top);
        const float sub = m_new == -INFINITY ? 0.0f : m_new;
        const float alpha = exp2_fast(m - sub);
        m = m_new;
        float sum = 0.0f;
        uint4 pop[2][2];      // P^T as the second product's B operand: [32-key block][half of it]
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            uint32_t pw[8];
#pragma unroll
            for (int v2 = 0; v2 < 8; ++v2) {
                float p0 = exp2_fast(s[kb][2 * v2] - sub), p1 = exp2_fast(s[kb][2 * v2 + 1] - sub);
                sum += p0 + p1;
                if constexpr (KIND >= 2) {     // the values' scales ride on the operand, not on the sum
                    p0 *= vs_lds[buf][32 * kb + 8 * ((2 * v2) / 4) + 4 * h + (2 * v2) % 4];
                    p1 *= vs_lds[buf][32 * kb + 8 * ((2 * v2 + 1) / 4) + 4 * h + (2 * v2 + 1) % 4];
                }
                pw[v2] = to_pair<F16>(p0, p1);
            }
            pop[kb][0] = make_uint4(pw[0], pw[1], pw[2], pw[3]);
            pop[kb][1] = make_uint4(pw[4], pw[5], pw[6], pw[7]);
        }
        l = __builtin_fmaf(l, alpha, sum);
        // wave-uniform: skip the rescale when no row's maximum moved (alpha == 1 everywhere)
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int v = 0; v < 16; ++v) o[nb][v] *= alpha;
        }
        // O^T += V^T P^T: the lane feeds V^T[dim 32 nb + n32][keys of its half] and its own probabilities.
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int row = 32 * nb + n32;
            const int sw = swz(row);
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int g0 = 8 * kb + 4 * half + h;
                    const uint2 lo = *reinterpret_cast<const uint2*>(&vl[row * BN + 4 * (g0 ^ sw)]);
                    const uint2 hi = *reinterpret_cast<const uint2*>(&vl[row * BN + 4 * ((g0 + 2) ^ sw)]);
                    o[nb] = mfma<F16>(make_uint4(lo.x, lo.y, hi.x, hi.y), pop[kb][half], o[nb]);
                }
            }
        }
        __syncthreads();          // every wavefront is done with this buffer; the other one is stored
    }
    // The two half-waves hold the same row's sums over different keys.
    l += __shfl_xor(l, 32);
    if (!live) return;
    if (a.sinks) {
        const Fold f = fold(m, l, a.sinks[head] * kLog2e, 1.0f);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int v = 0; v < 16; ++v) o[nb][v] *= f.keep;
        m = f.m, l = f.l;
    }
    const float inv = l != 0.0f ? v_mult / l : 0.0f;
    const int64_t at = (int64_t)(start + t) * a.o_st + (int64_t)head * a.o_sh;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) {
            const int d = 32 * nb + 8 * v4 + 4 * h;
            const float x0 = o[nb][4 * v4] * inv, x1 = o[nb][4 * v4 + 1] * inv, x2 = o[nb][4 * v4 + 2] * inv, x3 = o[nb][4 * v4 + 3] * inv;
            if (a.out_dtype == CRIT_PKV_F32) {
                *reinterpret_cast<float4*>(reinterpret_cast<float*>(a.out) + at + d) = make_float4(x0, x1, x2, x3);
            } else if (a.out_dtype == CRIT_PKV_BF16) {
                *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(a.out) + at + d) = make_uint2(pack_bf16(x0, x1), pack_bf16(x2, x3));
            } else {
                *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(a.out) + at + d) = make_uint2(pack_f16(x0, x1), pack_f16(x2, x3));
            }
        }
    }
    if (a.lse && h == 0) a.lse[(int64_t)(start + t) * a.hq + head] = l != 0.0f ? __builtin_fmaf(m, kLn2, __logf(l)) : -INFINITY;
}

template <int KIND, bool F16>
static int launch_d(const PrefillArgs& a, int d, dim3 grid, hipStream_t stream) {
    switch (d) {
        case 64: hipLaunchKernelGGL((prefill_kernel<KIND, F16, 64>), grid, dim3(256), 0, stream, a); break;
        case 128: hipLaunchKernelGGL((prefill_kernel<KIND, F16, 128>), grid, dim3(256), 0, stream, a); break;
        default: return CRIT_PKV_E_GEOMETRY;
    }
    return hip_code(hipGetLastError());
}

int launch_prefill(const crit_pkv_prefill_params* p, hipStream_t stream) {
    if (!p || !p->q || !p->key_pages || !p->value_pages || !p->positions || !p->out) return CRIT_PKV_E_NULL;
    if ((p->tables == nullptr) == (p->tables64 == nullptr)) return CRIT_PKV_E_NULL;
    if (p->kind < 0 || p->kind > 3) return CRIT_PKV_E_DTYPE;
    if (p->kind >= 2 && (!p->key_scales || !p->value_scales)) return CRIT_PKV_E_NULL;
    const bool f16 = p->page_dtype == CRIT_PKV_F16;
    if (f16 && p->kind != 0) return CRIT_PKV_E_DTYPE;
    if (p->out_dtype != CRIT_PKV_F32 && p->out_dtype != CRIT_PKV_BF16 && p->out_dtype != CRIT_PKV_F16) return CRIT_PKV_E_DTYPE;
    if (p->chunks < 1 || p->chunks > 65535 || p->max_count < 1 || p->kv_heads < 1 || p->kv_heads > 65535 || p->heads < 1 ||
        p->heads % p->kv_heads || p->page < 1 || p->table_width < 1 || p->sliding < 0)
        return CRIT_PKV_E_GEOMETRY;
    if (p->head_dim != 64 && p->head_dim != 128) return CRIT_PKV_E_GEOMETRY;
    const int out_align = p->out_dtype == CRIT_PKV_F32 ? 4 : 4;      // 4 elements per store either way
    if (p->q_stride_t % 8 || p->q_stride_h % 8 || p->out_stride_t % out_align || p->out_stride_h % out_align ||
        (reinterpret_cast<uintptr_t>(p->q) % 16) || (reinterpret_cast<uintptr_t>(p->out) % 16) ||
        (reinterpret_cast<uintptr_t>(p->key_pages) % 16) || (reinterpret_cast<uintptr_t>(p->value_pages) % 16))
        return CRIT_PKV_E_GEOMETRY;
    PrefillArgs a;
    a.q = reinterpret_cast<const uint8_t*>(p->q);
    a.kp = reinterpret_cast<const uint8_t*>(p->key_pages);
    a.vp = reinterpret_cast<const uint8_t*>(p->value_pages);
    a.ks = p->key_scales, a.vs = p->value_scales;
    a.hm = p->kind == 1 ? p->head_multipliers : nullptr;
    a.tables = p->tables, a.tables64 = p->tables64, a.table_rows = p->table_rows, a.starts = p->starts, a.counts = p->counts;
    a.positions = p->positions;
    a.out = p->out, a.lse = p->lse, a.sinks = p->sinks;
    a.q_st = p->q_stride_t, a.q_sh = p->q_stride_h, a.o_st = p->out_stride_t, a.o_sh = p->out_stride_h, a.tab_stride = p->table_stride;
    a.tab_width = p->table_width, a.chunks = p->chunks, a.max_count = p->max_count, a.hq = p->heads, a.hkv = p->kv_heads;
    a.g = p->heads / p->kv_heads;
    a.page = p->page;
    a.page_shift = -1;
    for (int s = 0; s < 31; ++s)
        if ((1 << s) == p->page) a.page_shift = s;
    a.sliding = p->sliding, a.out_dtype = p->out_dtype;
    a.sscale = p->scale * kLog2e, a.k_mult = p->key_multiplier, a.v_mult = p->value_multiplier;
    const int64_t tiles = ((int64_t)p->max_count * a.g + BM - 1) / BM;
    if (tiles > 0x7fffffff) return CRIT_PKV_E_GEOMETRY;
    const dim3 grid((unsigned)tiles, (unsigned)p->kv_heads, (unsigned)p->chunks);
    switch (p->kind) {
        case 0: return f16 ? launch_d<0, true>(a, p->head_dim, grid, stream) : launch_d<0, false>(a, p->head_dim, grid, stream);
        case 1: return launch_d<1, false>(a, p->head_dim, grid, stream);
        case 2: return launch_d<2, false>(a, p->head_dim, grid, stream);
        case 3: return launch_d<3, false>(a, p->head_dim, grid, stream);
    }
    return CRIT_PKV_E_DTYPE;
}

}   // namespace pkv
