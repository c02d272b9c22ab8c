// Pool bookkeeping on the device (gfx950): the slots of positions through the bound page tables, the move of an accepted
// draft-tree path's rows to consecutive positions, the copy of whole pages, a round's lengths and a step's buffers. Integer and byte work, HBM-bound where
// it is bound by anything: what the reference does with torch indexing (inference/attention-state/code/pages.py:646-684,
// 861-869), one launch each, nothing read on the host.
#include "pkv_launch.hpp"

namespace pkv {
namespace {

typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

struct Tables {
    const int32_t* tables;
    const int64_t* capacity;
    int64_t round_slots, table_stride;
    int table_pages, page;
    int64_t dump_slot;      // the dump page's first slot
};

// KVPool._slots_at for one position (pages.py:655-660).
__device__ __forceinline__ int64_t slot_at(const Tables& t, int64_t s, int64_t p) {
    if (s < 0 || s >= t.round_slots) return t.dump_slot;
    if (p < 0 || p >= t.capacity[s]) return t.dump_slot;
    int64_t entry = p / t.page;
    entry = entry > t.table_pages - 1 ? t.table_pages - 1 : entry;
    return (int64_t)t.tables[s * t.table_stride + entry] * t.page + p % t.page;
}

__global__ __launch_bounds__(256) void slots_kernel(Tables t, const int64_t* slots, const int64_t* rows,
                                                    const int64_t* positions, int64_t* out, int64_t n, int64_t n_slots) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    int64_t s;
    if (rows) {
        const int64_t r = rows[i];
        s = r >= 0 && r < n_slots ? slots[r] : -1;
    } else {
        s = slots[i];
    }
    out[i] = slot_at(t, s, positions[i]);
}

struct Stores {
    crit_pkv_store s[CRIT_PKV_MAX_STORES];
    int wide[CRIT_PKV_MAX_STORES];      // the store moves 16 bytes a lane (its base, stride and unit allow it), else 4
};

constexpr int kStageBytes = 16384;      // (with the lists: six workgroups a compute unit)

// One workgroup: one round row, one layer, one store. The kept columns' source and target slots are listed first; then
// the rows move through LDS a slice of their bytes at a time, every source of the slice read before a target is
// written (a target may be a later column's source: index_copy_(index_select()) reads them all first).
template <typename G>
__device__ __forceinline__ void move_rows(uint8_t* base, int64_t row_bytes, const int64_t* s_src, const int64_t* s_dst, int n,
                                          uint4* stage16) {
    G* stage = reinterpret_cast<G*>(stage16);
    const int tid = threadIdx.x;
    const int row_g = (int)(row_bytes / (int64_t)sizeof(G));
    int slice = (int)(kStageBytes / sizeof(G)) / n;
    slice = slice > row_g ? row_g : slice;
    for (int g0 = 0; g0 < row_g; g0 += slice) {
        const int w = row_g - g0 < slice ? row_g - g0 : slice;
        for (int i = tid; i < n * w; i += 256) {
            const int c = i / w, g = i - c * w;
            stage[i] = reinterpret_cast<const G*>(base + s_src[c] * row_bytes)[g0 + g];
        }
        __syncthreads();
        for (int i = tid; i < n * w; i += 256) {
            const int c = i / w, g = i - c * w;
            reinterpret_cast<G*>(base + s_dst[c] * row_bytes)[g0 + g] = stage[i];
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(256) void compact_kernel(Tables t, Stores stores, const int64_t* start, const int64_t* emitted,
                                                      const void* path, int path_is_32, int64_t path_stride, int width,
                                                      const int64_t* moved) {
    __shared__ int64_t s_src[CRIT_PKV_MAX_PATH], s_dst[CRIT_PKV_MAX_PATH];
    __shared__ int s_kept[4];
    __shared__ uint4 stage[kStageBytes / sizeof(uint4)];
    const int tid = threadIdx.x;
    const int64_t r = blockIdx.x;
    const int layer = blockIdx.y;
    const crit_pkv_store st = stores.s[blockIdx.z];
    if (moved[r] != 0) return;
    const int64_t first = start[r], count = emitted[r];
    int64_t src = 0, dst = 0;
    int keep = 0;
    if (tid < width && tid > 0 && tid < count) {
        const int64_t node = path_is_32 ? (int64_t) reinterpret_cast<const int32_t*>(path)[r * path_stride + tid]
                                        : reinterpret_cast<const int64_t*>(path)[r * path_stride + tid];
        if (node >= 0) {
            src = slot_at(t, r, first + node);
            dst = slot_at(t, r, first + tid);
            // A target past the slot's capacity is the dump page: nothing is moved there. The reference's index_copy_
            // leaves one of the rows sent there, which one is not defined; what is defined is that a SOURCE past the
            // capacity reads the dump page as it was before the move, and it stays so only if no row's workgroup
            // writes it meanwhile.
            keep = dst != t.dump_slot;
        }
    }
    // (a column's place in the list: the kept columns before it, counted a wavefront at a time)
    const unsigned long long kept = __ballot(keep);
    const int lane = tid & 63, wave = tid >> 6;
    if (lane == 0) s_kept[wave] = __popcll(kept);
    __syncthreads();
    int at = __popcll(kept & ((1ull << lane) - 1ull));
    for (int w = 0; w < wave; ++w) at += s_kept[w];
    if (keep) s_src[at] = src, s_dst[at] = dst;
    const int n = s_kept[0] + s_kept[1] + s_kept[2] + s_kept[3];
    __syncthreads();
    if (n == 0) return;
    uint8_t* base = reinterpret_cast<uint8_t*>(st.base) + (int64_t)layer * st.layer_stride;
    if (stores.wide[blockIdx.z])
        move_rows<uint4>(base, st.row_bytes, s_src, s_dst, n, stage);
    else
        move_rows<uint32_t>(base, st.row_bytes, s_src, s_dst, n, stage);
}

__global__ __launch_bounds__(256) void set_moved_kernel(int64_t* moved, int64_t rows) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < rows) moved[i] = 1;
}

// KVPool.start_round / the end of commit_round (pages.py:623-644), one thread a round row.
__global__ __launch_bounds__(256) void round_kernel(int64_t* lengths, int64_t* start, int64_t* moved, const int64_t* emitted,
                                                    const int64_t* frontier, int64_t rows, int commit) {
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= rows) return;
    if (commit) {
        lengths[r] = emitted[r] > 0 ? frontier[r] : start[r];
    } else {
        start[r] = lengths[r];
        if (moved) moved[r] = 0;
    }
}

struct StepArgs {
    const int64_t *lengths, *slot, *counts, *firsts;
    int64_t *d_slots, *positions_t, *rows_t;
    int32_t *starts_t, *d_rows, *d_starts, *d_counts;
    int64_t* d_firsts;
    int32_t *d_offsets, *d_tables;
    int64_t* totals;
    int64_t rows, d_tables_stride, step_tokens, step_rows, count_each, window;
    int dump;
};

__device__ __forceinline__ int64_t count_of(const StepArgs& a, int64_t r) {
    const int64_t c = a.counts ? a.counts[r] : a.count_each;
    return c < 0 ? 0 : c;
}

// A step's buffers. Workgroup b < rows is row b; workgroup rows + w is window entry w, which it empties if fewer window
// rows exist. Every workgroup adds up the rows before its own (all rows, for an entry): the counts are a few KiB that
// stay in cache, and no workgroup waits for another.
__global__ __launch_bounds__(256) void step_kernel(Tables t, StepArgs a) {
    __shared__ int64_t s_sum[4][3];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool is_row = (int64_t)blockIdx.x < a.rows;
    const int64_t r = is_row ? (int64_t)blockIdx.x : a.rows;      // rows before r are added up
    int64_t tokens = 0, windows = 0, window_tokens = 0;
    for (int64_t i = tid; i < r; i += 256) {
        const int64_t c = count_of(a, i);
        tokens += c;
        if (c <= a.window) windows += 1, window_tokens += c;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        tokens += __shfl_xor(tokens, o);
        windows += __shfl_xor(windows, o);
        window_tokens += __shfl_xor(window_tokens, o);
    }
    if (lane == 0) s_sum[wave][0] = tokens, s_sum[wave][1] = windows, s_sum[wave][2] = window_tokens;
    __syncthreads();
    tokens = s_sum[0][0] + s_sum[1][0] + s_sum[2][0] + s_sum[3][0];
    windows = s_sum[0][1] + s_sum[1][1] + s_sum[2][1] + s_sum[3][1];
    window_tokens = s_sum[0][2] + s_sum[1][2] + s_sum[2][2] + s_sum[3][2];
    if (!is_row) {
        const int64_t w = (int64_t)blockIdx.x - a.rows;
        if (w == 0 && tid == 0) {
            a.totals[0] = tokens, a.totals[1] = windows, a.totals[2] = window_tokens;
            a.totals[3] = tokens > a.step_tokens || windows > a.step_rows ? 1 : 0;
            if (a.starts_t) a.starts_t[a.rows] = (int32_t)tokens;
        }
        if (w < windows || w >= a.step_rows) return;
        if (tid == 0) {
            if (a.d_rows) a.d_rows[w] = (int32_t)w;
            a.d_starts[w] = 0, a.d_counts[w] = 0, a.d_firsts[w] = 0, a.d_offsets[w] = (int32_t)window_tokens;
        }
        for (int e = tid; e < t.table_pages; e += 256) a.d_tables[w * a.d_tables_stride + e] = a.dump;
        return;
    }
    const int64_t s = a.slot[r], count = count_of(a, r);
    const bool bound = s >= 0 && s < t.round_slots;
    const int64_t first = a.firsts ? a.firsts[r] : (bound ? a.lengths[s] : 0);
    if (tid == 0 && a.starts_t) a.starts_t[r] = (int32_t)tokens;
    for (int64_t j = tid; j < count; j += 256) {
        const int64_t i = tokens + j;
        if (i >= a.step_tokens) break;
        a.d_slots[i] = slot_at(t, s, first + j);
        if (a.positions_t) a.positions_t[i] = first + j;
        if (a.rows_t) a.rows_t[i] = r;
    }
    if (count > a.window || windows >= a.step_rows) return;
    const int64_t w = windows;
    if (tid == 0) {
        if (a.d_rows) a.d_rows[w] = (int32_t)w;
        a.d_starts[w] = (int32_t)tokens, a.d_counts[w] = (int32_t)count, a.d_firsts[w] = first;
        a.d_offsets[w] = (int32_t)window_tokens;
    }
    for (int e = tid; e < t.table_pages; e += 256)
        a.d_tables[w * a.d_tables_stride + e] = bound ? t.tables[s * t.table_stride + e] : a.dump;
}

// One workgroup: a piece of one page of one layer of one store; every load of a thread issued before its stores.
template <typename G>
__device__ __forceinline__ void copy_piece(uint8_t* base, int64_t page_bytes, int64_t from, int64_t to, int piece) {
    const G* src = reinterpret_cast<const G*>(base + from * page_bytes);
    G* dst = reinterpret_cast<G*>(base + to * page_bytes);
    const int64_t total = page_bytes / (int64_t)sizeof(G);
    const int64_t lo = (int64_t)piece * 1024;
    G held[4];      // (read once, written once: nontemporal both ways, the caches keep neither)
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int64_t i = lo + k * 256 + threadIdx.x;
        if (i < total) held[k] = __builtin_nontemporal_load(src + i);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int64_t i = lo + k * 256 + threadIdx.x;
        if (i < total) __builtin_nontemporal_store(held[k], dst + i);
    }
}

__global__ __launch_bounds__(256) void copy_pages_kernel(Stores stores, const int64_t* source, const int64_t* target, int page,
                                                         int pieces, int64_t pool_pages) {
    const int which = blockIdx.x / pieces, piece = blockIdx.x - which * pieces;
    const crit_pkv_store st = stores.s[blockIdx.z];
    const int64_t from = source[which], to = target[which];
    if (from < 0 || to < 0 || (pool_pages > 0 && (from >= pool_pages || to >= pool_pages))) return;
    uint8_t* base = reinterpret_cast<uint8_t*>(st.base) + (int64_t)blockIdx.y * st.layer_stride;
    if (stores.wide[blockIdx.z])
        copy_piece<u32x4>(base, st.row_bytes * page, from, to, piece);
    else
        copy_piece<uint32_t>(base, st.row_bytes * page, from, to, piece);
}

// Checks the stores and notes which of them move 16 bytes a lane (unit_rows: the rows that move together).
int take_stores(const crit_pkv_store* s, int n, int64_t unit_rows, Stores& out) {
    for (int i = 0; i < CRIT_PKV_MAX_STORES; ++i) out.s[i] = s[i < n ? i : 0], out.wide[i] = 0;
    for (int i = 0; i < n; ++i) {
        if (!s[i].base) return CRIT_PKV_E_NULL;
        if (s[i].row_bytes < 4 || s[i].row_bytes % 4 || s[i].layer_stride % 4 || s[i].layer_stride < 0 ||
            reinterpret_cast<uintptr_t>(s[i].base) % 4)
            return CRIT_PKV_E_GEOMETRY;
        out.wide[i] = (s[i].row_bytes * unit_rows) % 16 == 0 && s[i].layer_stride % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(s[i].base) % 16 == 0;
    }
    return 0;
}

int check_tables(const int32_t* tables, const int64_t* capacity, int64_t round_slots, int64_t table_stride, int table_pages,
                 int page, int dump) {
    if (!tables || !capacity) return CRIT_PKV_E_NULL;
    if (round_slots < 1 || table_pages < 1 || table_stride < table_pages || page < 1 || dump < 0) return CRIT_PKV_E_GEOMETRY;
    return 0;
}

}   // namespace

int launch_slots_at(const crit_pkv_slots_params* p, hipStream_t stream) {
    if (!p) return CRIT_PKV_E_NULL;
    if (p->n == 0) return 0;
    if (!p->slots || !p->positions || !p->out) return CRIT_PKV_E_NULL;
    if (const int bad = check_tables(p->round_tables, p->round_capacity, p->round_slots, p->table_stride, p->table_pages,
                                     p->page, p->dump))
        return bad;
    if (p->n < 0 || p->n > ((int64_t)1 << 31) * 255 || (p->rows && p->n_slots < 1)) return CRIT_PKV_E_GEOMETRY;
    const Tables t{p->round_tables, p->round_capacity, p->round_slots, p->table_stride, p->table_pages, p->page,
                   (int64_t)p->dump * p->page};
    hipLaunchKernelGGL(slots_kernel, dim3((unsigned)((p->n + 255) / 256)), dim3(256), 0, stream, t, p->slots, p->rows,
                       p->positions, p->out, p->n, p->n_slots);
    return (int)hipGetLastError();
}

int launch_compact(const crit_pkv_compact_params* p, hipStream_t stream) {
    if (!p) return CRIT_PKV_E_NULL;
    if (p->rows == 0) return 0;
    if (!p->start || !p->emitted || !p->path || !p->moved) return CRIT_PKV_E_NULL;
    if (const int bad = check_tables(p->round_tables, p->round_capacity, p->round_slots, p->table_stride, p->table_pages,
                                     p->page, p->dump))
        return bad;
    if (p->rows < 0 || p->rows > p->round_slots || p->rows > 0x7fffffff || p->width < 1 || p->width > CRIT_PKV_MAX_PATH ||
        p->path_stride < p->width || p->layers < 1 || p->layers > 65535 || p->n_stores < 1 || p->n_stores > CRIT_PKV_MAX_STORES)
        return CRIT_PKV_E_GEOMETRY;
    Stores stores;
    if (const int bad = take_stores(p->stores, p->n_stores, 1, stores)) return bad;
    const Tables t{p->round_tables, p->round_capacity, p->round_slots, p->table_stride, p->table_pages, p->page,
                   (int64_t)p->dump * p->page};
    const dim3 grid((unsigned)p->rows, (unsigned)p->layers, (unsigned)p->n_stores);
    hipLaunchKernelGGL(compact_kernel, grid, dim3(256), 0, stream, t, stores, p->start, p->emitted, p->path, p->path_is_32,
                       p->path_stride, p->width, p->moved);
    if (const hipError_t e = hipGetLastError()) return (int)e;
    hipLaunchKernelGGL(set_moved_kernel, dim3((unsigned)((p->rows + 255) / 256)), dim3(256), 0, stream, p->moved, p->rows);
    return (int)hipGetLastError();
}

int launch_copy_pages(const crit_pkv_copy_pages_params* p, hipStream_t stream) {
    if (!p) return CRIT_PKV_E_NULL;
    if (p->n == 0) return 0;
    if (!p->source || !p->target) return CRIT_PKV_E_NULL;
    if (p->n < 0 || p->pool_pages < 0 || p->page < 1 || p->layers < 1 || p->layers > 65535 || p->n_stores < 1 ||
        p->n_stores > CRIT_PKV_MAX_STORES)
        return CRIT_PKV_E_GEOMETRY;
    Stores stores;
    if (const int bad = take_stores(p->stores, p->n_stores, p->page, stores)) return bad;
    int64_t pieces = 1;      // 1,024 granules a workgroup: as many workgroups a page as the store that needs most
    for (int i = 0; i < p->n_stores; ++i) {
        const int64_t needs = (p->stores[i].row_bytes * p->page / (stores.wide[i] ? 16 : 4) + 1023) / 1024;
        pieces = needs > pieces ? needs : pieces;
    }
    if (pieces * p->n > 0x7fffffff) return CRIT_PKV_E_GEOMETRY;
    const dim3 grid((unsigned)(pieces * p->n), (unsigned)p->layers, (unsigned)p->n_stores);
    hipLaunchKernelGGL(copy_pages_kernel, grid, dim3(256), 0, stream, stores, p->source, p->target, p->page, (int)pieces,
                       p->pool_pages);
    return (int)hipGetLastError();
}

int launch_round(const crit_pkv_round_params* p, hipStream_t stream) {
    if (!p) return CRIT_PKV_E_NULL;
    if (p->rows == 0) return 0;
    if (!p->round_lengths || !p->start || (p->commit && (!p->emitted || !p->frontier))) return CRIT_PKV_E_NULL;
    if (p->rows < 0 || p->rows > ((int64_t)1 << 31) * 255) return CRIT_PKV_E_GEOMETRY;
    hipLaunchKernelGGL(round_kernel, dim3((unsigned)((p->rows + 255) / 256)), dim3(256), 0, stream, p->round_lengths, p->start,
                       p->moved, p->emitted, p->frontier, p->rows, p->commit);
    return (int)hipGetLastError();
}

int launch_step_buffers(const crit_pkv_step_params* p, hipStream_t stream) {
    if (!p) return CRIT_PKV_E_NULL;
    if (!p->slot || !p->d_slots || !p->d_starts || !p->d_counts || !p->d_firsts || !p->d_offsets || !p->d_tables || !p->totals ||
        (!p->round_lengths && !p->firsts))
        return CRIT_PKV_E_NULL;
    if (const int bad = check_tables(p->round_tables, p->round_capacity, p->round_slots, p->table_stride, p->table_pages,
                                     p->page, p->dump))
        return bad;
    if (p->rows < 0 || p->rows > 32768 || p->step_rows < 0 || p->step_rows > 32768 || p->step_tokens < 0 ||
        p->step_tokens > 0x7fffffff || p->d_tables_stride < p->table_pages || p->window < 0 || (!p->counts && p->count_each < 0))
        return CRIT_PKV_E_GEOMETRY;
    const Tables t{p->round_tables, p->round_capacity, p->round_slots, p->table_stride, p->table_pages, p->page,
                   (int64_t)p->dump * p->page};
    const StepArgs a{p->round_lengths, p->slot, p->counts, p->firsts, p->d_slots, p->positions_t, p->rows_t, p->starts_t,
                     p->d_rows, p->d_starts, p->d_counts, p->d_firsts, p->d_offsets, p->d_tables, p->totals, p->rows,
                     p->d_tables_stride, p->step_tokens, p->step_rows, p->count_each, p->window, p->dump};
    // (one workgroup a row, one a window entry, and at least the one that writes the totals)
    const int64_t grid = p->rows + (p->step_rows > 0 ? p->step_rows : 1);
    hipLaunchKernelGGL(step_kernel, dim3((unsigned)grid), dim3(256), 0, stream, t, a);
    return (int)hipGetLastError();
}

}   // namespace pkv
