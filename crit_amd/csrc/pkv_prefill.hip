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
#include "pkv_launch.hpp"
#include "pkv_prefill.hpp"

namespace pkv {

// RESUME: the launch that continues rows from their states over a chunk's fresh rows (PrefillArgs::mode 2; 16-bit only).
// IQK: INT8 pages with the first product in integers (the reference's int8_qk): each query row becomes INT8 codes at its
// own scale, the keys' codes go to LDS as they are, and S^T = K Q^T is v_mfma_i32_32x32x32_i8 (32 dims a step).
template <int KIND, bool F16, int D, int WAVES, bool RESUME = false, bool IQK = false>
__global__ __launch_bounds__(64 * WAVES, D == 256 ? 1 : 8 / WAVES) void prefill_kernel(PrefillArgs a) {
    static_assert(!RESUME || KIND == 0, "fresh rows are 16-bit");
    static_assert(!IQK || KIND == 3, "integer scores: INT8 pages");
    constexpr int KSTR8 = D + 16;       // IQK: K row stride in LDS (bytes)
    static_assert(D == 64 || D == 128 || D == 256, "head widths 64, 128, 256");
    static_assert(WAVES == 4 || (WAVES == 8 && D == 128), "eight wavefronts: 128-wide heads only");
    constexpr int NT = 64 * WAVES;      // threads of the workgroup
    constexpr int BMW = 32 * WAVES;     // query rows it holds
    constexpr int KS = D / 16;          // k-steps of the first product
    constexpr int NB = D / 32;          // 32-wide output blocks of the second product
    constexpr int KSTR = D + 8;         // K row stride in LDS (16-bit elements): 16 bytes of padding
    constexpr int EB = KIND == 0 ? 2 : 1;
    constexpr int CH = D * EB / 16;     // 16-byte chunks of one K or V row in the pages
    constexpr int KPASS = BN * CH / NT;    // passes of the workgroup over a K block, rows contiguous over lanes
    // V staging: a thread takes DPT dims (eight, or four where eight wavefronts share the block) of four adjacent keys;
    // D / DPT such pieces a key, 16 groups of four keys a block.
    constexpr int DPT = WAVES == 8 ? 4 : 8;
    constexpr int VC = D / DPT;         // pieces of one V row
    constexpr int VGROUPS = 16 * VC;    // (group of four keys, piece) pairs of a V block: the workgroup's threads, or half of them (D = 64)
    constexpr int VPASS = (VGROUPS + NT - 1) / NT;      // ... or twice them (D = 256): a thread then takes two pairs, NT apart
    // K blocks alternate between two buffers. V blocks too with four wavefronts; with eight, half of the wavefronts
    // multiply by a block's values one iteration after the other half (below), so V blocks go round three buffers.
    constexpr int VBUFS = WAVES == 8 ? 3 : 2;
    __shared__ __align__(16) uint16_t k_lds[2][BN * KSTR];
    __shared__ __align__(16) uint16_t v_lds[VBUFS][D * BN];
    __shared__ float ks_lds[2][BN], vs_lds[VBUFS][BN];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n32 = lane & 31, h = lane >> 5;
    // Workgroups go to the 8 XCDs round robin by linear id, and each XCD has its own L2: all tiles of one (chunk, KV
    // head) read the same keys, so they take ids of one residue mod 8 and share that XCD's L2. Later tiles see more
    // keys: they start first.
    const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
    const int group = xcd + 8 * (q / a.tiles);
    if (group >= a.hkv * a.chunks) return;
    const int tile = a.tiles - 1 - q % a.tiles;
    const int kvh = group % a.hkv, z = chunk_by_rank(a, group / a.hkv, lane);
    int count = a.max_count;
    if (a.counts) count = min(a.counts[z], a.max_count);
    if ((int64_t)tile * BMW >= (int64_t)count * a.g) return;
    const int start = a.starts ? a.starts[z] : 0;
    int64_t pos64 = a.positions[z];
    pos64 = pos64 < 0 ? 0 : (pos64 > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : pos64);
    const int pos = (int)pos64;
    // Positions from `first` on belong to the other launch of a chunk with fresh rows (between the chunk's position
    // and its end, as the reference clamps it).
    int first = 0;
    if (a.mode != 0) {
        int64_t f = a.firsts ? a.firsts[z] : pos64;
        f = f < pos64 ? pos64 : (f > pos64 + count ? pos64 + count : f);
        first = (int)f;
    }
    const int64_t trow = (int64_t)(a.table_rows ? a.table_rows[z] : z) * a.tab_stride;

    // This lane's query row.
    const int j = tile * BMW + wave * 32 + n32;
    const int t = j / a.g, head = kvh * a.g + j % a.g;
    const bool live = t < count;
    const int lim = live ? pos + t : -1;
    // 16-bit scores: the lane's B operand of k-step ks is dims 16 ks + 8 h .. + 7 of its row. Integer scores: of step
    // ks (32 dims) dims 32 ks + 16 h .. + 15, as codes; qreg[ks] for ks < D / 32 then holds 16 codes.
    uint4 qreg[KS];
    float q_scale = 1.0f;      // IQK: the row's scale, amax / 127
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        qreg[ks] = make_uint4(0, 0, 0, 0);
        if (live) {
            const int dim = IQK ? 32 * (ks / 2) + 16 * h + 8 * (ks % 2) : 16 * ks + 8 * h;
            qreg[ks] = *reinterpret_cast<const uint4*>(a.q + ((int64_t)(start + t) * a.q_st + (int64_t)head * a.q_sh + dim) * 2);
        }
    }
    if constexpr (IQK) {
        // Each query row to INT8 at its own scale (amax / 127, at least 1e-30), rounded half away from zero
        // (_kernels.py:637-643); the two half-waves hold the two halves of the row's dims.
        float x[KS][8];
        float amax = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const uint32_t w[4] = {qreg[ks].x, qreg[ks].y, qreg[ks].z, qreg[ks].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                x[ks][2 * i] = u2f(w[i] << 16), x[ks][2 * i + 1] = u2f(w[i] & 0xffff0000u);
                amax = __builtin_fmaxf(amax, __builtin_fmaxf(__builtin_fabsf(x[ks][2 * i]), __builtin_fabsf(x[ks][2 * i + 1])));
            }
        }
        amax = __builtin_fmaxf(amax, __shfl_xor(amax, 32));
        q_scale = __builtin_fmaxf(__fdiv_rn(amax, 127.0f), 1e-30f);
#pragma unroll
        for (int s2 = 0; s2 < KS / 2; ++s2) {
            uint32_t code[4];
#pragma unroll
            for (int wd = 0; wd < 4; ++wd) {
                uint32_t packed = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int e = 4 * wd + i;      // element 0 .. 15 of the step: registers 2 s2 (0 .. 7) and 2 s2 + 1 (8 .. 15)
                    const float f = __fdiv_rn(x[2 * s2 + e / 8][e % 8], q_scale);
                    const int c = (int)(f >= 0.0f ? f + 0.5f : f - 0.5f);      // (a NaN row gives codes of 0, as the cast does)
                    packed |= ((uint32_t)c & 0xffu) << (8 * i);
                }
                code[wd] = packed;
            }
            qreg[s2] = make_uint4(code[0], code[1], code[2], code[3]);
        }
    }
    // The lowest limit among the wavefront's live rows: key blocks wholly at or below it need no mask.
    int wave_lo = live ? lim : 0x7fffffff;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) wave_lo = min(wave_lo, __shfl_xor(wave_lo, o));
    wave_lo = __builtin_amdgcn_readfirstlane(wave_lo);
    float k_mult = a.k_mult, v_mult = a.v_mult;
    if (KIND == 1 && a.hm) k_mult = a.hm[kvh], v_mult = a.hm[a.hkv + kvh];
    const float sscale = a.sscale * (KIND == 1 ? k_mult : 1.0f) * q_scale;
    if (KIND != 1) v_mult = 1.0f;
    const int win = a.sliding;
    const float sabs = __builtin_fabsf(sscale);
    if (sscale < 0.0f && KIND < 2) {      // a negative scale: its sign goes into the queries, |scale| into the exponent
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            qreg[ks].x ^= 0x80008000u, qreg[ks].y ^= 0x80008000u, qreg[ks].z ^= 0x80008000u, qreg[ks].w ^= 0x80008000u;
        }
    }

    const int t_lo = tile * BMW / a.g;
    const int t_hi = min(count - 1, (tile * BMW + BMW - 1) / a.g);
    const int n_max = a.mode == 1 ? first - 1 : pos + count - 1;      // the last position whose row is read
    int kt_hi = (pos + t_hi) / BN;
    int kt_lo = 0;
    if (win > 0) kt_lo = max(0, pos + t_lo - win + 1) / BN;
    if (a.mode == 1) kt_hi = first > 0 ? min(kt_hi, (first - 1) / BN) : -1;
    if (RESUME) kt_lo = max(kt_lo, first / BN);
    const bool any_block = kt_hi >= kt_lo;      // (always with mode 0)
    // The lowest and highest position this launch reads for any row.
    const int cap = a.mode == 1 ? first - 1 : 0x3fffffff;
    const int floor_excl = RESUME ? first - 1 : -0x20000000;

    // A block's 64 keys map onto the 64 lanes: lane i looks up the page table entry and the slot of position 64 kt + i
    // (positions past the chunk's last written one read that one), every wavefront for itself, and a thread then takes
    // the slots of the rows it loads from the lanes that hold them (ds_bpermute). One 4-byte table load whatever the
    // table's type: an int64 entry's low word holds the page number (little endian). Slots fit 32 unsigned bits: a
    // row is at least 64 bytes and a pool at most the card's memory.
    const uint8_t* tab_row = (a.tables ? reinterpret_cast<const uint8_t*>(a.tables) : reinterpret_cast<const uint8_t*>(a.tables64)) +
                             (trow << (a.tables ? 2 : 3));
    const int tab_shift = a.tables ? 2 : 3;
    const uint32_t k_slot_bytes = a.k_slot_bytes, v_slot_bytes = a.v_slot_bytes;
    const uint8_t* kbase = a.kp + (int64_t)kvh * D * EB;
    const uint8_t* vbase = a.vp + (int64_t)kvh * D * EB;
    // Global -> registers -> LDS. K: rows contiguous over lanes. V: a thread takes eight dims of four adjacent keys and
    // stores them transposed as eight 8-byte groups (8-bit codes become 16-bit values on the way, exactly).
    // The page table entries of a block are fetched one block before its rows (load_entries, then take_slots, then load_k and load_v): a
    // row's address depends on its entry, and a wait on an entry would also wait on every row load issued before it.
    u32x4 kreg[KPASS], vreg[VPASS][4];      // vreg[vp][i]: key 4 kg + i of pass vp; 8-bit pages fill .x and .y only
    int ent = 0, inp = 0;
    float ksreg = 1.0f, vsreg = 1.0f;
    constexpr bool direct = RESUME;      // fresh rows: the chunk's tokens in order, no table (the launcher sets page = 1)
    auto load_entries = [&](int kt) __attribute__((always_inline)) {
        int n = kt * BN + lane;
        n = n < n_max ? n : n_max;
        uint32_t pidx = (__umulhi(a.page_magic, (uint32_t)n) + (uint32_t)n) >> a.page_l;
        const int in_page = n - (int)pidx * a.page;
        pidx = pidx < (uint32_t)a.tab_width ? pidx : (uint32_t)a.tab_width - 1u;
        const int got = *reinterpret_cast<const int*>(tab_row + ((direct ? 0u : pidx) << tab_shift));      // (unconditional: entry 0 when unused)
        ent = direct ? start + max(n - pos, 0) : got;
        inp = direct ? 0 : in_page;
    };
    // take_slots turns the entries into slots and hands every thread the slots of its rows; it runs during the second
    // product of the iteration before the loads that use them, so the exchange's latency passes behind the products
    // and load_k / load_v issue their row loads back to back.
    constexpr int NROW = KPASS + 4 * VPASS;
    uint32_t rowslot[NROW], myslot = 0;
    auto take_slots = [&]() __attribute__((always_inline)) {
        myslot = (uint32_t)ent * (uint32_t)a.page + (uint32_t)inp;
        static_for<KPASS>([&](auto pc) __attribute__((always_inline)) {
            constexpr int p = decltype(pc)::value;
            rowslot[p] = (uint32_t)__builtin_amdgcn_ds_bpermute(((p * NT + tid) / CH) << 2, (int)myslot);
        });
        static_for<4 * VPASS>([&](auto ic) __attribute__((always_inline)) {
            constexpr int vp = decltype(ic)::value / 4, i = decltype(ic)::value % 4;
            const int kg = (vp * NT + tid) % VGROUPS / VC;      // D = 64: the upper half of the workgroup repeats the lower
            rowslot[KPASS + 4 * vp + i] = (uint32_t)__builtin_amdgcn_ds_bpermute((4 * kg + i) << 2, (int)myslot);
        });
    };
    auto load_k = [&]() __attribute__((always_inline)) {
        const uint8_t* kthread = kbase + (tid % CH) * 16;
        static_for<KPASS>([&](auto pc) __attribute__((always_inline)) {
            constexpr int p = decltype(pc)::value;
            kreg[p] = *reinterpret_cast<const u32x4*>(kthread + (uint64_t)rowslot[p] * k_slot_bytes);
        });
        if constexpr (KIND >= 2) ksreg = a.ks[(uint64_t)myslot * a.hkv + kvh];
    };
    auto load_v = [&]() __attribute__((always_inline)) {
        static_for<4 * VPASS>([&](auto ic) __attribute__((always_inline)) {
            constexpr int vp = decltype(ic)::value / 4, i = decltype(ic)::value % 4;
            const uint8_t* vthread = vbase + ((vp * NT + tid) % VGROUPS % VC) * (DPT * EB);
            const uint8_t* row = vthread + (uint64_t)rowslot[KPASS + 4 * vp + i] * v_slot_bytes;
            if constexpr (DPT * EB == 16) {
                vreg[vp][i] = *reinterpret_cast<const u32x4*>(row);
            } else if constexpr (DPT * EB == 8) {
                const u32x2 w = *reinterpret_cast<const u32x2*>(row);
                vreg[vp][i].x = w.x, vreg[vp][i].y = w.y;
            } else {
                vreg[vp][i].x = *reinterpret_cast<const uint32_t*>(row);
            }
        });
        if constexpr (KIND >= 2) vsreg = a.vs[(uint64_t)myslot * a.hkv + kvh];
    };
    auto store_k = [&](int buf) __attribute__((always_inline)) {
        uint16_t* kl = k_lds[buf];
        static_for<KPASS>([&](auto pc) __attribute__((always_inline)) {
            constexpr int p = decltype(pc)::value;
            const int idx = p * NT + tid;
            const int kk = idx / CH, c = idx % CH;
            if constexpr (KIND == 0) {
                *reinterpret_cast<u32x4*>(&kl[kk * KSTR + c * 8]) = kreg[p];
            } else if constexpr (IQK) {
                *reinterpret_cast<u32x4*>(reinterpret_cast<uint8_t*>(kl) + kk * KSTR8 + c * 16) = kreg[p];
            } else {
                *reinterpret_cast<u32x4*>(&kl[kk * KSTR + c * 16]) = codes_to_bf16<KIND>(kreg[p].x, kreg[p].y);
                PKV_SB();      // one 16-byte group converted and stored at a time keeps the conversions' temporaries few
                *reinterpret_cast<u32x4*>(&kl[kk * KSTR + c * 16 + 8]) = codes_to_bf16<KIND>(kreg[p].z, kreg[p].w);
                PKV_SB();
            }
        });
        if constexpr (KIND >= 2) {
            if (tid < BN) ks_lds[buf][tid] = ksreg;
        }
    };
    auto store_v = [&](int buf) __attribute__((always_inline)) {
        // The thread's four keys x DPT dims as 16-bit pairs of adjacent dims (8-bit codes converted, exactly), then
        // transposed: dim row 8 c + i gets the four keys' values as one 8-byte group at the place v_place gives, byte
        // offset v_place(kg, 8 c) ^ (16 i), plus 128 i. A thread with four dims holds i = 4 up + 0 .. 3 of them: 64 up
        // goes into the XOR and 512 up into the sum (bits 7 to 9 of the first term are clear, so the sum carries nothing).
        uint8_t* vb = reinterpret_cast<uint8_t*>(v_lds[buf]);
        if constexpr (KIND >= 2) {
            if (tid < BN) vs_lds[buf][tid] = vsreg;
        }
        static_for<VPASS>([&](auto vpc) __attribute__((always_inline)) {
        constexpr int vp = decltype(vpc)::value;
        const int idx = (vp * NT + tid) % VGROUPS;      // repeated pairs store the same bytes twice
        const int kg = idx / VC, piece = idx % VC;
        const int c = piece / (8 / DPT), up = piece % (8 / DPT);
        const uint32_t v_write = ((uint32_t)v_place(kg, 8 * c) ^ (64u * (uint32_t)up)) + 512u * (uint32_t)up;
        static_for<DPT / 2>([&](auto jc) __attribute__((always_inline)) {
            constexpr int j = decltype(jc)::value;      // dims 2 j and 2 j + 1 of the thread's eight
            uint32_t w[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                if constexpr (KIND == 0) {
                    w[k] = vreg[vp][k][j];
                } else {
                    w[k] = code_pair<KIND, j % 2 == 1>(vreg[vp][k][j / 2]);
                }
            }
#pragma unroll
            for (int i = 2 * j; i < 2 * j + 2; ++i) {
                const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
                const uint32_t k01 = __builtin_amdgcn_perm(w[1], w[0], sel);
                const uint32_t k23 = __builtin_amdgcn_perm(w[3], w[2], sel);
                *reinterpret_cast<u32x2*>(vb + (v_write ^ (16u * i)) + 128 * i) = u32x2{k01, k23};
            }
            if constexpr (KIND != 0) PKV_SB();      // (as in store_k)
        });
        });
    };
    // Operand reads, two operands a step. K, step i: k-step i of both 32-key halves. V, step i: keys
    // 16 (i / (NB / 2)) .. + 15 of the 32-dim blocks 2 (i % (NB / 2)) and the next one.
    auto read_k = [&](const uint16_t* kl, auto ic, u32x4 (&dst)[2]) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if constexpr (IQK) {
                dst[kb] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint8_t*>(kl) + (32 * kb + n32) * KSTR8 + 32 * i + 16 * h);
            } else {
                dst[kb] = *reinterpret_cast<const u32x4*>(&kl[(32 * kb + n32) * KSTR + 16 * i + 8 * h]);
            }
        }
    };
    // Byte offset of the lane's V^T operand inside a buffer: row 32 nb + n32, the 16-byte slot of groups 4 g + h and
    // 4 g + 2 + h = v_place(4 g + h, 32 nb + n32) = v_read ^ (16 (2 g ^ 4 (nb & 1))) + 4096 nb.
    const uint32_t v_read = (uint32_t)v_place(h, n32);
    auto read_v = [&](const uint16_t* vl, auto ic, u32x4 (&dst)[2]) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        constexpr int g = i / (NB / 2);      // keys 16 g .. 16 g + 15: 32-key half g / 2, half of it g % 2
        const uint8_t* vb = reinterpret_cast<const uint8_t*>(vl);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int nb = 2 * (i % (NB / 2)) + j;
            const u32x4 w = *reinterpret_cast<const u32x4*>(vb + (v_read ^ (16u * ((2 * g) ^ (4 * (nb & 1))))) + 32 * BN * 2 * nb);
            dst[j] = w;
        }
    };

    f32x16 o[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[nb][v] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    if (RESUME && live) {
        const int64_t state_at = ((int64_t)(start + t) * a.hq + head) * (D + kStatePad);      // the state the launch over the pages left: this lane's dims, the row's maximum, its sum once
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
            for (int v4 = 0; v4 < 4; ++v4) {
                const float4 x = *reinterpret_cast<const float4*>(a.state + state_at + 32 * nb + 8 * v4 + 4 * h);
                o[nb][4 * v4] = x.x, o[nb][4 * v4 + 1] = x.y, o[nb][4 * v4 + 2] = x.z, o[nb][4 * v4 + 3] = x.w;
            }
        }
        m = a.state[state_at + D];
        l = h == 0 ? a.state[state_at + D + 1] : 0.0f;
    }

    // Double-buffered LDS, one barrier a block: block kt is multiplied from buffer kt & 1 while block kt + 1 (already
    // in registers) is stored into the other buffer and its registers are at once reloaded with block kt + 2 (a whole
    // iteration before they are stored); the slots of block kt + 3 and the table entries of block kt + 4 follow. Every
    // load of the loop is unconditional (past the last block it repeats the last one), so the compiler counts the
    // outstanding loads exactly instead of waiting for all of them.
    auto upto = [&](int kt) __attribute__((always_inline)) { return kt < kt_hi ? kt : kt_hi; };
    if (any_block) {
        load_entries(kt_lo);
        take_slots();
        load_k();
        load_v();
        load_entries(upto(kt_lo + 1));
        store_k(kt_lo & 1);
        store_v(WAVES == 8 ? 0 : kt_lo & 1);
        take_slots();
        load_k();
        load_v();
        load_entries(upto(kt_lo + 2));
        take_slots();
        load_entries(upto(kt_lo + 3));
        __syncthreads();
    }

    // A key block in three phases. scores: S^T = K Q^T on the matrix cores, with the staging of the next block in its
    // shadow. weigh: mask, running maximum, the first exponentials (vector work). values: O^T += V^T P^T on the matrix
    // cores, the remaining exponentials in its shadow.
    constexpr int RING = 3;      // operands are read RING - 1 steps before their products
    f32x16 s[2];
    u32x4 va[RING][2], pop[4];
    float alpha = 1.0f, sum = 0.0f, sub = 0.0f;
    const std::integral_constant<int, 0> c0;
    const std::integral_constant<int, 1> c1;
    // kt: the block; vnext: the V buffer block kt + 1 goes to.
    auto scores = [&](int kt, int vnext) __attribute__((always_inline)) {
        const int buf = kt & 1;
        const uint16_t* kl = k_lds[buf];
        // Two blocks of 32 keys x this wavefront's 32 rows. The operands of a step are read RING - 1 steps before it,
        // and the next block goes into the other LDS buffers (their readers passed the barrier) in the shadow of the
        // products.
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int v = 0; v < 16; ++v) s[kb][v] = 0.0f;
        u32x4 ka[RING][2];
        static_for<RING - 1>([&](auto ic) __attribute__((always_inline)) { read_k(kl, ic, ka[decltype(ic)::value]); });
        constexpr int KSTEPS = IQK ? D / 32 : KS;      // steps of 32 dims with integer scores, of 16 otherwise
        i32x16 si[2];
        if constexpr (IQK) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) si[kb][v] = 0;
        }
        PKV_PRIO(1);
        static_for<KSTEPS>([&](auto ic) __attribute__((always_inline)) {
            constexpr int i = decltype(ic)::value;
            if constexpr (i + RING - 1 < KSTEPS) read_k(kl, std::integral_constant<int, i + RING - 1>{}, ka[(i + RING - 1) % RING]);
            if constexpr (IQK) {
                const i32x4 qi = {(int)qreg[i].x, (int)qreg[i].y, (int)qreg[i].z, (int)qreg[i].w};
                si[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, ka[i % RING][0]), qi, si[0], 0, 0, 0);
                si[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, ka[i % RING][1]), qi, si[1], 0, 0, 0);
            } else {
                s[0] = mfma<F16>(ka[i % RING][0], qreg[i], s[0]);
                s[1] = mfma<F16>(ka[i % RING][1], qreg[i], s[1]);
            }
            if constexpr (i == 0) store_k(buf ^ 1), load_k();
            if constexpr (i == KSTEPS / 2 - 1) store_v(vnext), load_v();
            if constexpr (WAVES == 8 && i == KSTEPS - 2) {      // the slots of block kt + 3 for the next iteration's loads, the entries of kt + 4
                take_slots();
                load_entries(upto(kt + 4));
            }
            if constexpr (KIND != 0) PKV_SB();
        });
        if constexpr (IQK) {      // exact integer dot products of the codes; the rows' and keys' scales follow below
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) s[kb][v] = (float)si[kb][v];
        }
        // one product, then a share of the staging work (LDS reads of later operands, the stores' permutes and
        // writes, the row loads) in its shadow
        if constexpr (KIND == 0 && D != 256) {      // (8-bit pages: the conversions' temporaries make this order spill)
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * (RING - 1), 0);
            static_for<2 * KS>([&](auto) __attribute__((always_inline)) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            });
        }
        PKV_SB();
        PKV_PRIO(0);
        // With one scale for all keys (positive once its sign went into the queries) the maximum is taken over the raw
        // scores and the scale rides on the exponent's fused multiply-add; with per-key scales (row-scaled pages) each
        // score is scaled first. The lane holds keys 32 kb + 8 (v / 4) + 4 h + v % 4 of its own row.
        if constexpr (KIND >= 2) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) s[kb][v] *= sscale * ks_lds[buf][32 * kb + 8 * (v / 4) + 4 * h + v % 4];
        }
    };
    // P^T as the second product's B operand: pop[g] holds the probabilities of keys 16 g .. 16 g + 15 (32-key half
    // g / 2, half of it g % 2), four 16-bit pairs, taken two pairs at a time so that only the first two pairs'
    // exponentials run before the second product starts and the rest in the shadow of its matrix instructions.
    auto pairs = [&](int vbuf, auto gc, auto partc) __attribute__((always_inline)) {
        constexpr int g = decltype(gc)::value, part = decltype(partc)::value;
        constexpr int kb = g / 2, half = g % 2;
#pragma unroll
        for (int j = 2 * part; j < 2 * part + 2; ++j) {
            const int v = 8 * half + 2 * j;
            float p0, p1;
            if constexpr (KIND >= 2) {
                p0 = exp2_fast(s[kb][v] - sub), p1 = exp2_fast(s[kb][v + 1] - sub);
            } else {
                p0 = exp2_fast(__builtin_fmaf(s[kb][v], sabs, -sub)), p1 = exp2_fast(__builtin_fmaf(s[kb][v + 1], sabs, -sub));
            }
            sum += p0 + p1;
            if constexpr (KIND >= 2) {     // the values' scales ride on the operand, not on the sum
                p0 *= vs_lds[vbuf][32 * kb + 8 * (v / 4) + 4 * h + v % 4];
                p1 *= vs_lds[vbuf][32 * kb + 8 * ((v + 1) / 4) + 4 * h + (v + 1) % 4];
            }
            pop[g][j] = to_pair<F16>(p0, p1);
        }
    };
    // MASK: 0 = every key of the block is visible to every row of the workgroup, 1 = causal limit and sliding window.
    auto weigh = [&](int kt, int vbuf, auto mask_c) __attribute__((always_inline)) {
        constexpr int MASK = decltype(mask_c)::value;
        const uint16_t* vl = v_lds[vbuf];
        static_for<RING - 1>([&](auto ic) __attribute__((always_inline)) { read_v(vl, ic, va[decltype(ic)::value]); });
        PKV_SB();
        if constexpr (MASK > 0) {
            // key 32 kb + 8 (v / 4) + v % 4 + 4 h is visible iff that constant is in (rel_lo, rel]
            const int rel = min(lim, cap) - kt * BN - 4 * h;
            const int rel_lo = max(win > 0 ? lim - win : -0x20000000, floor_excl) - kt * BN - 4 * h;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int c = 32 * kb + 8 * (v / 4) + v % 4;
                    const bool vis = c <= rel && c > rel_lo;
                    s[kb][v] = vis ? s[kb][v] : -INFINITY;
                }
            }
        }
        float top = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                top = __builtin_fmaxf(top, s[kb][v]);
            }
        }
        if constexpr (KIND < 2) top = top == -INFINITY ? -INFINITY : top * sabs;
        {      // the two half-waves meet by one lane swap in the vector pipe (a shuffle is a round trip through the LDS crossbar)
            const int w = (int)f2u(top);
            const auto both = __builtin_amdgcn_permlane32_swap(w, w, false, false);
            top = __builtin_fmaxf(u2f((uint32_t)both[0]), u2f((uint32_t)both[1]));
        }
        const float m_new = top > m + kMaxSlack ? top : m;
        sub = m_new == -INFINITY ? 0.0f : m_new;
        alpha = exp2_fast(m - sub);
        m = m_new;
        sum = 0.0f;
        pairs(vbuf, c0, c0);
        pairs(vbuf, c0, c1);
        // wave-uniform: skip the rescale when no row's maximum moved (alpha == 1 everywhere)
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
            asm volatile("s_nop 0");      // pins the branch: an unconditional rescale by 1 is what the optimiser would make of it
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int v = 0; v < 16; ++v) o[nb][v] *= alpha;
        }
        PKV_SB();
    };
    // The lane feeds V^T[dim 32 nb + n32][keys of its half] and its own probabilities. The second half's exponentials
    // run in the shadow of the first half's products.
    auto values = [&](int kt, int vbuf) __attribute__((always_inline)) {
        const uint16_t* vl = v_lds[vbuf];
        PKV_PRIO(1);
        constexpr int VSTEPS = 2 * NB;
        static_for<VSTEPS>([&](auto ic) __attribute__((always_inline)) {
            constexpr int i = decltype(ic)::value;
            constexpr int g = i / (NB / 2), nb = 2 * (i % (NB / 2));
            if constexpr (i + RING - 1 < VSTEPS) read_v(vl, std::integral_constant<int, i + RING - 1>{}, va[(i + RING - 1) % RING]);
            o[nb] = mfma<F16>(va[i % RING][0], pop[g], o[nb]);
            o[nb + 1] = mfma<F16>(va[i % RING][1], pop[g], o[nb + 1]);
            // steps 0 .. 5 take the pairs of pop[1], pop[2], pop[3] in order, each a step (D = 128) or more (D = 64:
            // two at a time) before the step that multiplies by them
            if constexpr (NB >= 4) {
                if constexpr (i < 6) pairs(vbuf, std::integral_constant<int, 1 + i / 2>{}, std::integral_constant<int, i % 2>{});
            } else {
                if constexpr (i == 0) pairs(vbuf, c1, c0), pairs(vbuf, c1, c1);
                if constexpr (i == 1) pairs(vbuf, std::integral_constant<int, 2>{}, c0), pairs(vbuf, std::integral_constant<int, 2>{}, c1);
                if constexpr (i == 2) pairs(vbuf, std::integral_constant<int, 3>{}, c0), pairs(vbuf, std::integral_constant<int, 3>{}, c1);
            }
            if constexpr (WAVES == 4 && i == VSTEPS - 2) {      // the slots of block kt + 3 for the next iteration's loads, the entries of kt + 4
                take_slots();
                load_entries(upto(kt + 4));
            }
            PKV_SB();
        });
        PKV_PRIO(0);
        l = __builtin_fmaf(l, alpha, sum);
    };
    // Blocks wholly visible to every row of the workgroup first (none under a sliding window), then the masked ones.
    int kt_full = win > 0 ? kt_lo : max(kt_lo, min(kt_hi + 1, (pos + t_lo + 1) / BN));
    if (a.mode == 1) kt_full = max(kt_lo, min(kt_full, first / BN));      // blocks wholly below the first fresh position
    // A resuming launch's first block may begin below the first fresh position: blocks up to kt_lead take the mask too.
    int kt_lead = kt_lo;
    if (RESUME && win == 0) kt_lead = min(max(kt_lo, (first + BN - 1) / BN), kt_hi + 1);
    kt_full = max(kt_full, kt_lead);
    if (!any_block) {
        // no position of this launch for these rows: the state passes through
    } else if constexpr (WAVES == 4) {
        int kt = kt_lo;
        if constexpr (RESUME) {
            for (; kt < kt_lead; ++kt) {
                scores(kt, (kt & 1) ^ 1), weigh(kt, kt & 1, c1), values(kt, kt & 1);
                __syncthreads();
            }
        }
        for (; kt < kt_full; ++kt) {
            scores(kt, (kt & 1) ^ 1), weigh(kt, kt & 1, c0), values(kt, kt & 1);
            __syncthreads();          // every wavefront is done with this buffer; the other one is stored
        }
        for (; kt <= kt_hi; ++kt) {
            scores(kt, (kt & 1) ^ 1), weigh(kt, kt & 1, c1), values(kt, kt & 1);
            __syncthreads();
        }
    } else {
        // Eight wavefronts, two a SIMD, and the barrier keeps them in step: were both of a SIMD in the same phase, its
        // matrix pipe would idle while they weigh and its vector pipe while they multiply. So wavefronts 4 to 7 run a
        // block's phases rotated by one iteration: between two barriers they weigh and multiply the values of block
        // kt - 1 and then take the scores of block kt, while wavefronts 0 to 3 take the scores of block kt, weigh it
        // and multiply its values: whenever one of a SIMD's two is in a matrix phase the other is in vector work or in the
        // other matrix phase's complement. Both kinds stage block kt + 1 during their scores of block kt, so a K buffer
        // is read in one iteration by all (two buffers) and a V buffer in two successive ones (three).
        auto after = [](int b) { return b == 2 ? 0 : b + 1; };
        const bool behind = __builtin_amdgcn_readfirstlane(wave >> 2) != 0;
        if (!behind) {
            int vcur = 0, kt = kt_lo;
            if constexpr (RESUME) {
                for (; kt < kt_lead; ++kt) {
                    scores(kt, after(vcur)), weigh(kt, vcur, c1), values(kt, vcur);
                    __syncthreads();
                    vcur = after(vcur);
                }
            }
            for (; kt < kt_full; ++kt) {
                scores(kt, after(vcur)), weigh(kt, vcur, c0), values(kt, vcur);
                __syncthreads();
                vcur = after(vcur);
            }
            for (; kt <= kt_hi; ++kt) {
                scores(kt, after(vcur)), weigh(kt, vcur, c1), values(kt, vcur);
                __syncthreads();
                vcur = after(vcur);
            }
        } else {
            // iteration kt weighs block kt - 1: masked while that block is below kt_lead or from kt_full on
            scores(kt_lo, 1);
            __syncthreads();
            int vprev = 0, vcur = 1, kt = kt_lo + 1;
            if constexpr (RESUME) {
                for (; kt <= min(kt_lead, kt_hi); ++kt) {
                    weigh(kt - 1, vprev, c1), values(kt - 1, vprev), scores(kt, after(vcur));
                    __syncthreads();
                    vprev = vcur, vcur = after(vcur);
                }
            }
            for (; kt <= min(kt_full, kt_hi); ++kt) {
                weigh(kt - 1, vprev, c0), values(kt - 1, vprev), scores(kt, after(vcur));
                __syncthreads();
                vprev = vcur, vcur = after(vcur);
            }
            for (; kt <= kt_hi; ++kt) {
                weigh(kt - 1, vprev, c1), values(kt - 1, vprev), scores(kt, after(vcur));
                __syncthreads();
                vprev = vcur, vcur = after(vcur);
            }
            weigh(kt_hi, vprev, c1), values(kt_hi, vprev);      // (a mask over a wholly visible block changes nothing)
        }
    }
    // The two half-waves hold the same row's sums over different keys.
    l += __shfl_xor(l, 32);
    if (!live) return;
    if (a.mode == 1) {
        const int64_t state_at = ((int64_t)(start + t) * a.hq + head) * (D + kStatePad);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
            for (int v4 = 0; v4 < 4; ++v4) {
                // (the values' one multiplier, which a launch of its own applies with the final division, goes in here:
                // the fresh rows that follow count as given)
                *reinterpret_cast<float4*>(a.state + state_at + 32 * nb + 8 * v4 + 4 * h) =
                    make_float4(o[nb][4 * v4] * v_mult, o[nb][4 * v4 + 1] * v_mult, o[nb][4 * v4 + 2] * v_mult, o[nb][4 * v4 + 3] * v_mult);
            }
        }
        if (h == 0) a.state[state_at + D] = m, a.state[state_at + D + 1] = l;
        return;
    }
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

template <int KIND, bool F16, bool RESUME = false, bool IQK = false>
static int launch_d(const PrefillArgs& a, int d, bool wide, dim3 grid, hipStream_t stream) {
    switch (d) {
        case 64: hipLaunchKernelGGL((prefill_kernel<KIND, F16, 64, 4, RESUME, IQK>), grid, dim3(256), 0, stream, a); break;
        case 256:      // (one workgroup a compute unit: 133 KB of LDS, about 300 registers; integer scores at 64 and 128 only)
            if constexpr (IQK) return CRIT_PKV_E_GEOMETRY;
            else hipLaunchKernelGGL((prefill_kernel<KIND, F16, 256, 4, RESUME, false>), grid, dim3(256), 0, stream, a);
            break;
        case 128:
            if constexpr (!RESUME) {
                if (wide) {
                    hipLaunchKernelGGL((prefill_kernel<KIND, F16, 128, 8, RESUME, IQK>), grid, dim3(512), 0, stream, a);
                    break;
                }
            }
            {
                hipLaunchKernelGGL((prefill_kernel<KIND, F16, 128, 4, RESUME, IQK>), grid, dim3(256), 0, stream, a);
            }
            break;
        default: return CRIT_PKV_E_GEOMETRY;
    }
    return hip_code(hipGetLastError());
}

// One launch: the grid for the shape the launch takes, then the kernel of its kind.
static int launch_one(PrefillArgs a, int kind, bool f16, int head_dim, int kv_heads, int chunks, int max_count, hipStream_t stream) {
    // 128-wide heads: eight wavefronts on 256 rows stage each key block once for twice the rows, which pays where the
    // launch still has a workgroup or more for every compute unit.
    const int64_t groups8 = ((int64_t)kv_heads * chunks + 7) / 8;
    int64_t tiles = ((int64_t)max_count * a.g + 2 * BM - 1) / (2 * BM);
    // (The launch that resumes rows over their fresh positions is short and takes the four-wavefront shape: with its
    // three loops per wavefront group the eight-wavefront one spills.)
    const bool wide = head_dim == 128 && a.mode != 2 && tiles * kv_heads * chunks >= compute_units();
    if (!wide) tiles = ((int64_t)max_count * a.g + BM - 1) / BM;
    if (tiles * groups8 * 8 > 0x7fffffff) return CRIT_PKV_E_GEOMETRY;
    a.tiles = (int)tiles;
    const dim3 grid((unsigned)(tiles * groups8 * 8));
    switch (kind) {
        case 0:
            if (a.mode == 2) return f16 ? launch_d<0, true, true>(a, head_dim, wide, grid, stream) : launch_d<0, false, true>(a, head_dim, wide, grid, stream);
            return f16 ? launch_d<0, true>(a, head_dim, wide, grid, stream) : launch_d<0, false>(a, head_dim, wide, grid, stream);
        case 1: return launch_d<1, false>(a, head_dim, wide, grid, stream);
        case 2: return launch_d<2, false>(a, head_dim, wide, grid, stream);
        case 3:
            if (a.iqk) return launch_d<3, false, false, true>(a, head_dim, wide, grid, stream);
            return launch_d<3, false>(a, head_dim, wide, grid, stream);
    }
    return CRIT_PKV_E_DTYPE;
}

int launch_prefill(const crit_pkv_prefill_params* p, hipStream_t stream) {
    if (!p || !p->q || !p->key_pages || !p->value_pages || !p->positions || !p->out) return CRIT_PKV_E_NULL;
    if ((p->tables == nullptr) == (p->tables64 == nullptr)) return CRIT_PKV_E_NULL;
    if (p->kind < 0 || p->kind > 3) return CRIT_PKV_E_DTYPE;
    if (p->kind >= 2 && (!p->key_scales || !p->value_scales)) return CRIT_PKV_E_NULL;
    if (p->int8_qk && p->kind != 3) return CRIT_PKV_E_DTYPE;
    const bool f16 = p->page_dtype == CRIT_PKV_F16;
    if (f16 && p->kind != 0) return CRIT_PKV_E_DTYPE;
    if (p->out_dtype != CRIT_PKV_F32 && p->out_dtype != CRIT_PKV_BF16 && p->out_dtype != CRIT_PKV_F16) return CRIT_PKV_E_DTYPE;
    if (p->chunks < 1 || p->chunks > 65535 || p->max_count < 1 || p->max_count > (1 << 30) || p->kv_heads < 1 || p->kv_heads > 65535 || p->heads < 1 ||
        p->heads % p->kv_heads || p->page < 1 || p->table_width < 1 || p->sliding < 0)
        return CRIT_PKV_E_GEOMETRY;
    if (p->head_dim != 64 && p->head_dim != 128 && p->head_dim != 256) return CRIT_PKV_E_GEOMETRY;
    if (p->head_dim == 256 && p->int8_qk) return CRIT_PKV_E_GEOMETRY;
    const int out_align = p->out_dtype == CRIT_PKV_F32 ? 4 : 4;      // 4 elements per store either way
    if (p->q_stride_t % 8 || p->q_stride_h % 8 || p->out_stride_t % out_align || p->out_stride_h % out_align ||
        (reinterpret_cast<uintptr_t>(p->q) % 16) || (reinterpret_cast<uintptr_t>(p->out) % 16) ||
        (reinterpret_cast<uintptr_t>(p->key_pages) % 16) || (reinterpret_cast<uintptr_t>(p->value_pages) % 16))
        return CRIT_PKV_E_GEOMETRY;
    const bool fresh = p->fresh_keys != nullptr || p->fresh_values != nullptr;
    if (fresh) {
        if (!p->fresh_keys || !p->fresh_values || !p->fresh_state) return CRIT_PKV_E_NULL;
        const int64_t row = (int64_t)p->kv_heads * p->head_dim;
        if (p->fresh_stride_k < row || p->fresh_stride_v < row || p->fresh_stride_k % 8 || p->fresh_stride_v % 8 ||
            p->fresh_stride_k > 0x3fffffff || p->fresh_stride_v > 0x3fffffff ||
            (reinterpret_cast<uintptr_t>(p->fresh_keys) % 16) || (reinterpret_cast<uintptr_t>(p->fresh_values) % 16) ||
            (reinterpret_cast<uintptr_t>(p->fresh_state) % 16))
            return CRIT_PKV_E_GEOMETRY;
    }
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
    a.page_l = 0;
    while ((1ll << a.page_l) < p->page) ++a.page_l;
    a.page_magic = (uint32_t)((((1ull << a.page_l) - (uint64_t)p->page) << 32) / (uint64_t)p->page + 1);
    a.sliding = p->sliding, a.out_dtype = p->out_dtype;
    a.sscale = p->scale * kLog2e, a.k_mult = p->key_multiplier, a.v_mult = p->value_multiplier;
    a.firsts = nullptr, a.state = nullptr, a.mode = 0;
    a.iqk = p->int8_qk != 0;
    a.k_slot_bytes = a.v_slot_bytes = (uint32_t)p->kv_heads * p->head_dim * (p->kind == 0 ? 2 : 1);
    a.tiles = 0;
    if (!fresh) return launch_one(a, p->kind, f16, p->head_dim, p->kv_heads, p->chunks, p->max_count, stream);
    // The positions below each chunk's first fresh one from the pages, then the rest from the fresh rows (16-bit, in
    // q's type, no scales), through the rows' states.
    a.firsts = p->fresh_firsts, a.state = p->fresh_state, a.mode = 1;
    const int err = launch_one(a, p->kind, f16, p->head_dim, p->kv_heads, p->chunks, p->max_count, stream);
    if (err != 0) return err;
    a.mode = 2;
    a.kp = reinterpret_cast<const uint8_t*>(p->fresh_keys), a.vp = reinterpret_cast<const uint8_t*>(p->fresh_values);
    a.k_slot_bytes = (uint32_t)(p->fresh_stride_k * 2), a.v_slot_bytes = (uint32_t)(p->fresh_stride_v * 2);
    a.ks = a.vs = a.hm = nullptr;
    a.k_mult = a.v_mult = 1.0f;
    a.page = 1, a.page_l = 0, a.page_magic = 1;
    a.iqk = 0;      // (fresh rows are multiplied in q's type, as the reference's are)
    return launch_one(a, 0, f16, p->head_dim, p->kv_heads, p->chunks, p->max_count, stream);
}

}   // namespace pkv
