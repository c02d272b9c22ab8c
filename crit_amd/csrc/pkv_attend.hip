// Host side of the decode / verify-window launches (argument checks, grid, the choice of kernel) and the small
// kernels around the split launch: the merge of the partitions, the merge of shard partials, a streaming-read probe.
#include <atomic>

#include "pkv_attend_args.hpp"
#include "pkv_launch.hpp"

namespace pkv {

int launch_attend_bf16(const AttendArgs& a, int lpr, int qr, bool fused, bool page16, dim3 grid, hipStream_t stream);
int launch_attend_f16(const AttendArgs& a, int lpr, int qr, bool fused, bool page16, dim3 grid, hipStream_t stream);
int launch_attend_fp8(const AttendArgs& a, int lpr, int qr, bool fused, bool page16, dim3 grid, hipStream_t stream);
int launch_attend_fp8row(const AttendArgs& a, int lpr, int qr, bool fused, bool page16, dim3 grid, hipStream_t stream);
int launch_attend_int8(const AttendArgs& a, int lpr, int qr, bool fused, bool page16, dim3 grid, hipStream_t stream);

// One wavefront per (column, head, row): folds the partitions that hold the column's positions, in order.
// Lane `at`'s value of x (at: the same in every lane).
PKV_DEV float lane_value(float x, int at) { return u2f((uint32_t)__builtin_amdgcn_readlane((int)f2u(x), at)); }

template <int DV>
__global__ __launch_bounds__(64) void merge_kernel(AttendArgs a) {
    constexpr int EPL = DV < 64 ? 1 : DV / 64;      // (value rows narrower than a wavefront: the lanes past them idle)
    const int c = blockIdx.x, head = blockIdx.y, r = blockIdx.z;
    const int lane = DV < 64 ? min((int)threadIdx.x, DV - 1) : (int)threadIdx.x;
    int count = a.columns;
    if (a.counts) count = min(a.counts[r], a.columns);
    if (c >= count) return;
    int64_t first = a.firsts[r];
    first = first < 0 ? 0 : (first > (int64_t)0x3fffffff ? (int64_t)0x3fffffff : first);
    const int64_t seen = min(first + c + 1, (int64_t)a.max_keys);
    // (32-bit: seen <= max_keys; with block lists the partitions divide the list's run, the same for every column)
    const uint32_t run = a.blocks ? (uint32_t)a.listed_keys : (uint32_t)seen;
    const int nb = (int)min((uint32_t)a.parts, (run + (uint32_t)a.piece - 1u) / (uint32_t)a.piece);
    const int64_t prow = a.offsets ? (int64_t)(a.offsets[r] - a.offsets[0]) : (int64_t)r * a.columns;
    const int64_t at = ((prow + c) * a.hq + head) * a.parts;
    float M = -INFINITY, L = 0.0f, A[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) A[e] = 0.0f;
    // Folded strictly in partition order (the fused launch folds the same way: fold()). Few partitions (an ordinary
    // decode row): their states loaded 8 at a time so the loads overlap, then folded one by one.
    if (nb <= 8) {
        float pm[8], pl[8], po[8][EPL];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int b = u < nb ? u : nb - 1;
            pm[u] = a.pm[at + b], pl[u] = a.pl[at + b];
#pragma unroll
            for (int e = 0; e < EPL; ++e) po[u][e] = a.po[(at + b) * DV + e * 64 + lane];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (u < nb) {
                const Fold f = fold(M, L, pm[u], pl[u]);
#pragma unroll
                for (int e = 0; e < EPL; ++e) A[e] = __builtin_fmaf(A[e], f.keep, po[u][e] * f.take);
                M = f.m, L = f.l;
            }
        }
    } else {
        // Many partitions (a long row's hundreds): a fold's maximum, its two exponentials and the product l * take
        // depend only on the maxima before it, so a batch of U partitions takes them on U lanes at once, the same
        // operations on the same values as fold() one by one: the running maximum as a prefix maximum over the lanes
        // (exact in any order), then keep, take and l * take a lane each. What stays in order is one fused
        // multiply-add for the sum and one multiply and one fused multiply-add a value dim, their factors read from
        // the lane that holds them. The next batch's states are loaded while this one is folded.
        constexpr int U = EPL > 2 ? 16 : 32;
        float po[2][U][EPL], pm_next, pl_next;
        auto load_scalars = [&](int b0) __attribute__((always_inline)) {
            const int b = min(b0 + ((int)threadIdx.x & (U - 1)), nb - 1);      // (the thread's own place: `lane` is clamped to the value row)
            pm_next = a.pm[at + b], pl_next = a.pl[at + b];
        };
        auto load_values = [&](int b0, float (&dst)[U][EPL]) __attribute__((always_inline)) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int b = min(b0 + u, nb - 1);
#pragma unroll
                for (int e = 0; e < EPL; ++e) dst[u][e] = a.po[(at + b) * DV + e * 64 + lane];
            }
        };
        auto fold_batch = [&](int b0, float pm, float pl, const float (&val)[U][EPL]) __attribute__((always_inline)) {
            const int u_lane = (int)threadIdx.x & (U - 1);
            if (b0 + u_lane >= nb) pm = -INFINITY, pl = 0.0f;      // (lanes past the last partition are not folded below)
            float upto = pm;      // the maximum of this batch's partitions up to the lane's
#pragma unroll
            for (int o = 1; o < U; o <<= 1) {
                const float other = __shfl_up(upto, o, U);
                if (u_lane >= o) upto = __builtin_fmaxf(upto, other);
            }
            const float m_new = __builtin_fmaxf(M, upto);
            float m_old = __shfl_up(m_new, 1, U);
            if (u_lane == 0) m_old = M;
            const float sub = m_new == -INFINITY ? 0.0f : m_new;
            const float keep = exp2_fast(m_old - sub), take = exp2_fast(pm - sub);
            const float l_take = pl * take;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (b0 + u < nb) {
                    const float k_u = lane_value(keep, u), t_u = lane_value(take, u);
                    L = __builtin_fmaf(L, k_u, lane_value(l_take, u));
#pragma unroll
                    for (int e = 0; e < EPL; ++e) A[e] = __builtin_fmaf(A[e], k_u, val[u][e] * t_u);
                }
            }
            M = lane_value(m_new, min(nb - b0, U) - 1);
        };
        load_scalars(0);
        load_values(0, po[0]);
        for (int b0 = 0;;) {
            float pm = pm_next, pl = pl_next;
            load_scalars(b0 + U);      // (past the last partition the loads repeat it and are not folded)
            load_values(b0 + U, po[1]);
            fold_batch(b0, pm, pl, po[0]);
            b0 += U;
            if (b0 >= nb) break;
            pm = pm_next, pl = pl_next;
            load_scalars(b0 + U);
            load_values(b0 + U, po[0]);
            fold_batch(b0, pm, pl, po[1]);
            b0 += U;
            if (b0 >= nb) break;
        }
    }
    if (a.sinks) {
        const Fold f = fold(M, L, a.sinks[head] * kLog2e, 1.0f);
#pragma unroll
        for (int e = 0; e < EPL; ++e) A[e] *= f.keep;
        M = f.m, L = f.l;
    }
    const int64_t token = a.starts[r] + c;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
        const float o = L != 0.0f ? A[e] / L : 0.0f;
        if (DV >= 64 || (int)threadIdx.x < DV) store_out(a.out, a.out_dtype, token * a.o_st + (int64_t)head * a.o_sh + e * 64 + lane, o);
    }
    if (a.lse && threadIdx.x == 0) a.lse[token * a.hq + head] = L != 0.0f ? __builtin_fmaf(M, kLn2, __logf(L)) : -INFINITY;
}

// Shard merge: outs [parts][rows][DV], lses [parts][rows] (natural log) -> out FP32, lse; one wavefront per row.
template <int IN>
__global__ __launch_bounds__(64) void shard_merge_kernel(crit_pkv_merge_params p) {
    const int64_t row = blockIdx.x;
    const int lane = threadIdx.x;
    float top = -INFINITY;
    for (int i = 0; i < p.parts; ++i) top = __builtin_fmaxf(top, p.lses[(int64_t)i * p.rows + row]);
    const float sub = top == -INFINITY ? 0.0f : top;
    float total = 0.0f;
    for (int i = 0; i < p.parts; ++i) {
        const float x = p.lses[(int64_t)i * p.rows + row];
        total += x == -INFINITY ? 0.0f : __expf(x - sub);
    }
    for (int d = lane; d < p.value_dim; d += 64) {
        float acc = 0.0f;
        for (int i = 0; i < p.parts; ++i) {
            const float x = p.lses[(int64_t)i * p.rows + row];
            const float w = x == -INFINITY ? 0.0f : __expf(x - sub);
            const int64_t at = ((int64_t)i * p.rows + row) * p.value_dim + d;
            float v;
            if constexpr (IN == CRIT_PKV_F32) v = reinterpret_cast<const float*>(p.outs)[at];
            else if constexpr (IN == CRIT_PKV_BF16) v = u2f((uint32_t)reinterpret_cast<const uint16_t*>(p.outs)[at] << 16);
            else v = (float)reinterpret_cast<const _Float16*>(p.outs)[at];
            acc = __builtin_fmaf(w, v, acc);
        }
        p.out[row * p.value_dim + d] = total > 0.0f ? acc / total : 0.0f;
    }
    if (lane == 0) p.lse[row] = total > 0.0f ? sub + __logf(total) : -INFINITY;
}

__global__ __launch_bounds__(256) void stream_read_kernel(const uint4* data, int64_t vecs, float* sink) {
    uint32_t acc = 0;
    const int64_t stride = (int64_t)gridDim.x * 256 * 4;
    int64_t i = (int64_t)blockIdx.x * 256 * 4 + threadIdx.x;
    // Whole passes: four loads a thread, none under a condition, so all four are in flight together.
    for (; i + 768 < vecs; i += stride) {
        const u32x4* p = reinterpret_cast<const u32x4*>(data) + i;
        const u32x4 v0 = __builtin_nontemporal_load(p), v1 = __builtin_nontemporal_load(p + 256);
        const u32x4 v2 = __builtin_nontemporal_load(p + 512), v3 = __builtin_nontemporal_load(p + 768);
        acc ^= v0.x ^ v0.y ^ v0.z ^ v0.w ^ v1.x ^ v1.y ^ v1.z ^ v1.w ^ v2.x ^ v2.y ^ v2.z ^ v2.w ^ v3.x ^ v3.y ^ v3.z ^ v3.w;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {      // the last, partial pass of the workgroup that holds the end
        if (i + 256 * k < vecs) {
            const uint4 v = data[i + 256 * k];
            acc ^= v.x ^ v.y ^ v.z ^ v.w;
        }
    }
    if (acc == 0x12345678u) sink[threadIdx.x & 63] = 1.0f;    // keeps the loads alive; practically never taken
}

int launch_stream_read(const void* data, int64_t bytes, float* sink, hipStream_t stream) {
    if (!data || !sink) return CRIT_PKV_E_NULL;
    if (bytes < 0 || bytes % 16) return CRIT_PKV_E_GEOMETRY;
    hipLaunchKernelGGL(stream_read_kernel, dim3(256 * 16), dim3(256), 0, stream, reinterpret_cast<const uint4*>(data), bytes / 16, sink);
    return hip_code(hipGetLastError());
}

int launch_merge(const crit_pkv_merge_params* p, hipStream_t stream) {
    if (!p || !p->outs || !p->lses || !p->out || !p->lse) return CRIT_PKV_E_NULL;
    if (p->rows < 0 || p->parts < 1 || p->value_dim < 1) return CRIT_PKV_E_GEOMETRY;
    if (p->rows == 0) return 0;
    const dim3 grid((unsigned)p->rows);
    switch (p->in_dtype) {
        case CRIT_PKV_F32: hipLaunchKernelGGL((shard_merge_kernel<CRIT_PKV_F32>), grid, dim3(64), 0, stream, *p); break;
        case CRIT_PKV_BF16: hipLaunchKernelGGL((shard_merge_kernel<CRIT_PKV_BF16>), grid, dim3(64), 0, stream, *p); break;
        case CRIT_PKV_F16: hipLaunchKernelGGL((shard_merge_kernel<CRIT_PKV_F16>), grid, dim3(64), 0, stream, *p); break;
        default: return CRIT_PKV_E_DTYPE;
    }
    return hip_code(hipGetLastError());
}

// The tile heights the kernels are built for. A tile taller than a launch's rows computes rows nobody stores; a row's
// bits do not depend on the height of the tile it sits in.
static int pick_qr(int live_rows) {
    static const int choices[] = {1, 2, 4, 8};
    for (int c : choices)
        if (live_rows <= c) return c;
    return 8;
}

// -- compute units of the current device (cached: the query is a driver call) ----------------------------------------------
namespace {
constexpr int kMaxDevices = 64;
std::atomic<int> g_cus[kMaxDevices];      // 0: not asked yet
}   // namespace

int compute_units() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
    int n = g_cus[dev].load(std::memory_order_relaxed);
    if (n <= 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        g_cus[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// check_only: every refusal the launch can make is made, nothing is queued on the stream.
static int launch_attend_checked(const crit_pkv_attend_params* p, hipStream_t stream, bool check_only) {
    if (!p || !p->q || !p->value_pages || !p->tables || !p->rows || !p->starts || !p->firsts || !p->out) return CRIT_PKV_E_NULL;
    const bool derive = p->derive_table != nullptr;      // keys derived from the value rows: no key pages, no key scales
    if (!derive && !p->key_pages) return CRIT_PKV_E_NULL;
    if (p->kind < 0 || p->kind > 3) return CRIT_PKV_E_DTYPE;
    if (p->kind >= 2 && ((!derive && !p->key_scales) || !p->value_scales)) return CRIT_PKV_E_NULL;
    const bool f16 = p->page_dtype == CRIT_PKV_F16;
    if (f16 && p->kind != 0) return CRIT_PKV_E_DTYPE;
    if (p->out_dtype != CRIT_PKV_F32 && p->out_dtype != CRIT_PKV_BF16 && p->out_dtype != CRIT_PKV_F16) return CRIT_PKV_E_DTYPE;
    if (p->n_rows < 1 || p->columns < 1 || p->columns > CRIT_PKV_MAX_COLUMNS || p->kv_heads < 1 || p->heads < 1 ||
        p->heads % p->kv_heads || p->page < 1 || p->table_width < 1 || p->sliding < 0)
        return CRIT_PKV_E_GEOMETRY;
    auto width_ok = [](int d) { return d == 16 || d == 32 || d == 64 || d == 128 || d == 256; };
    if (!width_ok(p->head_dim) || !width_ok(p->value_dim)) return CRIT_PKV_E_GEOMETRY;
    if (p->q_stride_t % 8 || p->q_stride_h % 8 || (reinterpret_cast<uintptr_t>(p->q) % 16) ||
        (reinterpret_cast<uintptr_t>(p->key_pages) % 16) || (reinterpret_cast<uintptr_t>(p->value_pages) % 16))
        return CRIT_PKV_E_GEOMETRY;
    if (derive) {      // one row is key and value: one width; any even rotary width up to it
        if (p->head_dim != p->value_dim || p->derive_rot < 2 || p->derive_rot % 2 || p->derive_rot > p->head_dim ||
            !(p->derive_eps >= 0.0f) || p->blocks || p->fresh_keys)
            return CRIT_PKV_E_GEOMETRY;      // (fresh rows come as values only: their keys are derived too)
    }
    // INT8 queries against INT8 keys (prefill's int8_qk for the chunks it reads as window rows): the fused launch
    if (p->int8_qk && (p->kind != 3 || derive || p->blocks || !p->fused)) return p->kind != 3 ? CRIT_PKV_E_DTYPE : CRIT_PKV_E_GEOMETRY;
    const int lpr = (p->head_dim > p->value_dim ? p->head_dim : p->value_dim) / 8;      // lanes that hold the wider row
    const bool wide128 = p->head_dim == 128 && p->value_dim == 128;
    const bool wide256 = p->head_dim == 256 && p->value_dim == 256;      // (the matrix-core kernel's second width: two halves of 128)
    const int sp = 4 * (64 / lpr);
    if (p->partitions < 1 || p->partitions > 65535 || p->piece < 1 || p->piece % sp) return CRIT_PKV_E_WORKSPACE;
    if (!p->fused && (!p->partial_out || !p->partial_max || !p->partial_sum)) return CRIT_PKV_E_WORKSPACE;
    if (p->parents && p->parents64) return CRIT_PKV_E_NULL;
    if (p->blocks) {
        if (p->fused || p->sliding) return CRIT_PKV_E_GEOMETRY;
        if (p->blocks_k < 1 || p->blocks_k > kMaxListedBlocks || p->block_size < 1 || p->blocks_stride < p->blocks_k ||
            (int64_t)p->blocks_k * p->block_size > 0x3fffffff)
            return CRIT_PKV_E_GEOMETRY;
    }
    if ((p->parents || p->parents64) && p->columns > 64) return CRIT_PKV_E_GEOMETRY;      // an ancestor set is a 64-bit mask
    const bool fresh = p->fresh_keys != nullptr || p->fresh_values != nullptr;
    if (fresh) {
        if ((!p->fresh_keys && !derive) || !p->fresh_values || !p->fresh_shifts || !p->fresh_firsts) return CRIT_PKV_E_NULL;
        if (p->blocks) return CRIT_PKV_E_GEOMETRY;      // (block lists read the pages only, as the reference's)
        const int64_t row = (int64_t)p->kv_heads * p->head_dim, row_v = (int64_t)p->kv_heads * p->value_dim;
        if (p->fresh_rows < 1 || p->fresh_stride_v < row_v || p->fresh_stride_v % 8 || (reinterpret_cast<uintptr_t>(p->fresh_values) % 16))
            return CRIT_PKV_E_GEOMETRY;
        if (!derive && (p->fresh_stride_k < row || p->fresh_stride_k % 8 || (reinterpret_cast<uintptr_t>(p->fresh_keys) % 16)))
            return CRIT_PKV_E_GEOMETRY;
    }
    AttendArgs a;
    a.q = reinterpret_cast<const uint8_t*>(p->q);
    a.kp = reinterpret_cast<const uint8_t*>(p->key_pages);
    a.vp = reinterpret_cast<const uint8_t*>(p->value_pages);
    a.ks = p->key_scales, a.vs = p->value_scales;
    a.hm = p->kind == 1 ? p->head_multipliers : nullptr;
    a.tables = p->tables, a.rows = reinterpret_cast<const int32_t*>(p->rows), a.rows_step = p->rows_are_64 ? 2 : 1, a.starts = p->starts, a.counts = p->counts, a.firsts = p->firsts, a.offsets = p->offsets;
    a.po = p->partial_out, a.pm = p->partial_max, a.pl = p->partial_sum;
    a.out = p->out, a.lse = p->lse, a.sinks = p->sinks;
    a.parents = p->parents, a.parents64 = p->parents64;
    a.blocks = p->blocks, a.blocks_stride = p->blocks_stride, a.blocks_k = p->blocks_k, a.block_size = p->block_size;
    a.fk = reinterpret_cast<const uint8_t*>(p->fresh_keys), a.fv = reinterpret_cast<const uint8_t*>(p->fresh_values);
    a.f_shifts = p->fresh_shifts, a.f_firsts = p->fresh_firsts;
    a.f_stride_k = p->fresh_stride_k, a.f_stride_v = p->fresh_stride_v, a.f_rows = p->fresh_rows;
    a.f_per_row = p->fresh_per_row ? 1 : 0;
    a.derive_table = p->derive_table, a.derive_eps = p->derive_eps, a.derive_rot = p->derive_rot;
    a.derive_weighted = p->derive_weighted ? 1 : 0;
    a.iqk = p->int8_qk ? 1 : 0;
    a.listed_keys = p->blocks ? p->blocks_k * p->block_size : 0;
    a.block_div = make_div32(p->blocks ? (uint32_t)p->block_size : 1u);
    a.q_st = p->q_stride_t, a.q_sh = p->q_stride_h, a.o_st = p->out_stride_t, a.o_sh = p->out_stride_h, a.tab_stride = p->table_stride;
    a.tab_width = p->table_width, a.n_rows = p->n_rows, a.columns = p->columns, a.hq = p->heads, a.hkv = p->kv_heads;
    a.g = p->heads / p->kv_heads;
    a.dk = p->head_dim, a.dv = p->value_dim;
    a.page = p->page;
    a.page_shift = -1;
    for (int s = 0; s < 31; ++s)
        if ((1 << s) == p->page) a.page_shift = s;
    a.parts = p->partitions, a.piece = p->piece, a.sliding = p->sliding, a.out_dtype = p->out_dtype;
    a.sscale = p->scale * kLog2e, a.k_mult = p->key_multiplier, a.v_mult = p->value_multiplier;
    // 64-wide heads over an even number of KV heads: pairs of adjacent heads go through the bandwidth kernel as
    // 128-wide ones (what decides is the cache's geometry and the call's kind, never the launch's size)
    a.narrow = (p->head_dim == 64 && p->value_dim == 64 && p->kv_heads % 2 == 0 && !derive && !p->blocks && !a.iqk &&
                !(p->fresh_keys || p->fresh_values) && p->page % 16 == 0 && a.page_shift >= 4 &&
                (int64_t)p->partitions * p->piece <= 0x3fffffff && p->piece % 16 == 0) ? 1 : 0;
    if (a.narrow) a.hkv = p->kv_heads / 2, a.g *= 2, a.dk = a.dv = 128;
    const int live_rows = p->columns * a.g;
    int qr = pick_qr(live_rows);
    if (p->blocks) {      // a tile of one column's rows: the largest tile height that divides the group
        qr = a.g % 4 == 0 ? 4 : 1;      // (the block-list kernels are built for tiles of 1 and 4 rows)
    }
    // The generic kernel's variants that read fresh rows or derive their keys are built for tiles of 2 and 8 rows.
    if (fresh || derive || a.iqk) qr = qr <= 2 ? 2 : 8;      // (so is the one with INT8 queries)
    if (derive && p->head_dim != 64 && p->head_dim != 128) qr = 8;      // (derived keys at the other widths: tiles of 8 only)
    // The 128-wide kernel serves two adjacent KV heads per wavefront where the head count is even, so every position
    // is read in segments of two rows (512 bytes of 16-bit pages, 256 of 8-bit ones): measured best on MI355X against
    // one and four heads. Fixed by the cache's geometry, never by the launch: a column's bits depend on it.
    // (block lists of blocks that are a multiple of 16 positions walk their lists in the 128-wide kernel, others in
    // the generic one, each position looked up on its own)
    const bool fast_lists = p->blocks && wide128 && p->page % 16 == 0 && p->block_size % 16 == 0;
    const bool page16 = p->page % 16 == 0 && !p->blocks && !fresh;      // (rows with fresh positions take the generic kernel)
    a.heads_per_wave = 1;
    // The bandwidth kernel walks pages that are powers of two from 16 positions up, in positions below 2^31; other
    // multiples of 16 take the generic kernel. (block lists of blocks that are a multiple of 16: their own variant)
    const bool pow2_page = a.page_shift >= 4 && (int64_t)p->partitions * p->piece <= 0x3fffffff;
    a.fast128 = a.narrow || (!derive && !a.iqk && (((wide128 || wide256) && page16 && pow2_page && p->piece % 16 == 0) || fast_lists));      // (derived keys: the generic kernel)
    if (a.fast128 && (wide128 || a.narrow) && a.hkv % 2 == 0) a.heads_per_wave = 2;
    // Query rows a tile holds: the generic and block-list kernels' tile height; 16 a wavefront's heads share in the
    // bandwidth kernel (matrix tiles of 16 columns).
    const int tile_rows = a.fast128 && !p->blocks ? 16 / a.heads_per_wave : qr;
    a.tiles = (live_rows + tile_rows - 1) / tile_rows;
    // Windows of several tiles of 128-wide heads over 16-bit pages, split launch: a workgroup holds four tiles (one
    // workgroup a compute unit), or the two of a window of two (two workgroups still, with two dozen registers in
    // scratch outside the steps), and reads the rows once for all of them. A tile's bits are the same however many
    // share a workgroup, so this may follow the launch. Measured on MI355X (32 / 8 heads, 64 rows ~U[1024, 8192]): 4
    // columns 383 -> 288 us, 5 columns 519 -> 424, 8 columns 676 -> 480; one row of 32,768: 55 -> 45, 72 -> 56 and 91 ->
    // 62. Not taken where it measured slower: four tiles of 8-bit pages (8 columns 376 -> 334 us but 5 columns 279 ->
    // 302, one row 55 -> 92: the converted rows' steps are too long a chain for one wavefront a SIMD).
    a.query_tiles = 1;
    if (a.fast128 && !p->blocks && !p->fused && wide128 && p->kind == 0 && a.tiles >= 2) {
        a.query_tiles = a.tiles >= 3 ? 4 : 2;
        a.tiles = (a.tiles + a.query_tiles - 1) / a.query_tiles;
    }
    // 8-bit pages: two tiles a workgroup, two workgroups a compute unit still (FP8 in 242-252 registers; the row-scaled
    // kinds with two dozen in scratch outside the steps). 64 rows, 4 / 5 / 8 columns: FP8 207 -> 147, 279 -> 214, 376 ->
    // 230 us, INT8 224 -> 167, 307 -> 264, 428 -> 287 us; one row of 32,768 (FP8): 54 -> 52 and 64 -> 52 us, but a pair
    // alone (4 columns) 40 -> 51 us, so a window of two tiles pairs them only in launches that fill the card.
    if (a.fast128 && !p->blocks && !p->fused && wide128 && p->kind >= 1 && a.tiles >= 2) {
        const int64_t apart = (int64_t)p->n_rows * (p->kv_heads / a.heads_per_wave) * a.tiles * p->partitions;
        if (a.tiles >= 3 || apart > (int64_t)compute_units() * 2) {
            a.query_tiles = 2;
            a.tiles = (a.tiles + a.query_tiles - 1) / a.query_tiles;
        }
    }
    // 256-wide heads: pairs of tiles with one step in flight a wavefront instead of two (with two, 56-85 registers went
    // to scratch and 64 rows x 4 columns took 554 us against 443 apart; with one, 24 / 2 heads x 256 bf16, 64 rows, 2 / 4
    // / 5 / 8 columns: 287 -> 232, 445 -> 410, 569 -> 452, 856 -> 676 us; one row of 200,000: 255 -> 146 and 344 -> 237).
    if (a.fast128 && !p->blocks && !p->fused && wide256 && a.tiles >= 2) {
        a.query_tiles = 2;
        a.tiles = (a.tiles + a.query_tiles - 1) / a.query_tiles;
    }
    const int64_t gx = (int64_t)p->n_rows * (a.hkv / a.heads_per_wave) * a.tiles;
    if (gx > 0x7fffffff) return CRIT_PKV_E_GEOMETRY;
    // Positions past the page tables do not exist: partitions that could only hold such pieces are not launched.
    const int64_t table_keys = (int64_t)p->table_width * p->page;
    a.max_keys = (int)(table_keys < 0x3fffffff ? table_keys : 0x3fffffff);
    const int64_t live_parts = ((p->blocks ? (int64_t)a.listed_keys : (int64_t)a.max_keys) + (int64_t)p->piece - 1) / p->piece;
    const unsigned gy = (unsigned)(live_parts < p->partitions ? live_parts : p->partitions);
    const dim3 grid((unsigned)gx, p->fused ? 1u : gy);
    a.units_x = a.units_y = 0;
    // The unit-pulling launches draw their units from the caller's two counters; without them units are dealt in turn.
    a.ticket = p->launch_state;
    if (reinterpret_cast<uintptr_t>(p->launch_state) % 8) return CRIT_PKV_E_GEOMETRY;
    if (a.fast128 && compute_units() < 1) return CRIT_PKV_E_GEOMETRY;
    auto split = [&](bool fused) -> int {
        switch (p->kind) {
            case 0: return f16 ? launch_attend_f16(a, lpr, qr, fused, page16, grid, stream)
                               : launch_attend_bf16(a, lpr, qr, fused, page16, grid, stream);
            case 1: return launch_attend_fp8(a, lpr, qr, fused, page16, grid, stream);
            case 2: return launch_attend_fp8row(a, lpr, qr, fused, page16, grid, stream);
            case 3: return launch_attend_int8(a, lpr, qr, fused, page16, grid, stream);
        }
        return CRIT_PKV_E_DTYPE;
    };
    if (!p->fused && p->phases != 1 && (p->heads > 65535 || p->n_rows > 65535)) return CRIT_PKV_E_GEOMETRY;      // (the merge's grid)
    if (check_only) return 0;
    int rc = 0;
    if (p->fused) return split(true);
    if (p->phases != 2) rc = split(false);
    if (rc || p->phases == 1) return rc;
    const dim3 mgrid((unsigned)p->columns, (unsigned)p->heads, (unsigned)p->n_rows);
    switch (p->value_dim) {
        case 16: hipLaunchKernelGGL((merge_kernel<16>), mgrid, dim3(64), 0, stream, a); break;
        case 32: hipLaunchKernelGGL((merge_kernel<32>), mgrid, dim3(64), 0, stream, a); break;
        case 64: hipLaunchKernelGGL((merge_kernel<64>), mgrid, dim3(64), 0, stream, a); break;
        case 128: hipLaunchKernelGGL((merge_kernel<128>), mgrid, dim3(64), 0, stream, a); break;
        case 256: hipLaunchKernelGGL((merge_kernel<256>), mgrid, dim3(64), 0, stream, a); break;
    }
    return hip_code(hipGetLastError());
}

int launch_attend(const crit_pkv_attend_params* p, hipStream_t stream) { return launch_attend_checked(p, stream, false); }

// -- the entry point that allocates nothing ------------------------------------------------------------------------------
// The split launch's partials and its two counters in memory the library itself holds: a file-scope device array, one
// copy per GPU at its own address (looked up once per device, with that device current). Every call on a GPU shares
// that GPU's array.
static __device__ __align__(256) unsigned char scratch[CRIT_PKV_STATIC_SCRATCH_BYTES];

namespace {
constexpr int64_t kScratchHead = 256;      // the counters' share of the array; the partials follow
std::atomic<unsigned char*> g_scratch[kMaxDevices];

unsigned char* scratch_of_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    unsigned char* ptr = g_scratch[dev].load(std::memory_order_acquire);
    if (!ptr) {
        void* found = nullptr;
        if (hipGetSymbolAddress(&found, HIP_SYMBOL(scratch)) != hipSuccess || !found) return nullptr;
        ptr = static_cast<unsigned char*>(found);
        g_scratch[dev].store(ptr, std::memory_order_release);
    }
    return ptr;
}
}   // namespace

__global__ __launch_bounds__(64) void clear_counters_kernel(unsigned* counters) {
    if (threadIdx.x < 2) counters[threadIdx.x] = 0u;
}

int launch_attend_static(const crit_pkv_attend_params* p, hipStream_t stream) {
    if (!p) return CRIT_PKV_E_NULL;
    if (p->n_rows < 1 || p->columns < 1 || p->heads < 1 || p->partitions < 1 || p->value_dim < 1) return CRIT_PKV_E_GEOMETRY;
    // The partial rows a launch may write: every row's columns (rows packed by offsets take fewer).
    const int64_t states = (int64_t)p->n_rows * p->columns * p->heads * p->partitions;
    const int64_t need = p->fused ? 0 : states * ((int64_t)p->value_dim + 2) * (int64_t)sizeof(float);
    if (states > (int64_t)1 << 40 || kScratchHead + need > (int64_t)CRIT_PKV_STATIC_SCRATCH_BYTES) return CRIT_PKV_E_SCRATCH;
    unsigned char* base = scratch_of_current_device();
    if (!base) return CRIT_PKV_E_SCRATCH;
    crit_pkv_attend_params q = *p;
    q.launch_state = reinterpret_cast<uint32_t*>(base);
    float* partials = reinterpret_cast<float*>(base + kScratchHead);
    q.partial_out = p->fused ? nullptr : partials;
    q.partial_max = p->fused ? nullptr : partials + states * p->value_dim;
    q.partial_sum = p->fused ? nullptr : partials + states * ((int64_t)p->value_dim + 1);
    // A launch that would be refused queues nothing: the clear below touches counters that every stream of this GPU
    // shares, so it must not run for a call that is not going to launch.
    const int refused = launch_attend_checked(&q, stream, true);
    if (refused) return refused;
    // The counters start at zero whatever the last call left (a fill kernel: a captured graph replays it as it is).
    hipLaunchKernelGGL(clear_counters_kernel, dim3(1), dim3(64), 0, stream, reinterpret_cast<unsigned*>(base));
    const int rc = hip_code(hipGetLastError());
    if (rc) return rc;
    return launch_attend(&q, stream);
}

}   // namespace pkv
