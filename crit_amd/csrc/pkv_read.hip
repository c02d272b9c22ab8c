// Rows of a layer read back dequantised (gfx950): what KVPool.gather and KVPool.rows_at do with index_select, a cast and
// a multiply (inference/attention-state/code/pages.py:455-493), in one launch for keys and values. HBM-bound: a thread
// takes 8 or 16 elements of one (row, head) (16 bytes of a page where the head width allows it) and stores them in the output's
// type; value = float(code) * scale in FP32, rounded once to the output's type.
#include "pkv_common.hpp"
#include "pkv_launch.hpp"

namespace pkv {
namespace {

struct ReadArgs {
    const uint8_t* pages[2];      // keys, values
    const float* scales[2];       // row-scaled kinds: [slots][kv_heads]
    const float* head_mult;       // optional [2][kv_heads], kind FP8
    float mult[2];
    void* out[2];
    const int64_t* slots;         // [n], or null: through the table
    const int32_t* table;
    const int64_t* table64;
    int64_t n, pool_slots;        // pool_slots: a slot at or past it reads as zeros (0: not checked)
    int hkv, dim[2], page, kind, f16_pages, out_dtype;
};

// E elements a thread: 8 (16 bytes of a 16-bit page, 8 of an 8-bit page) or 16 codes of an 8-bit page (16 bytes), which
// the launcher takes for 16-bit outputs when the head widths allow it (262,144 rows of FP8 pages to BF16: 5.2 TB/s of
// bytes read and written against 3.7). Rows are read once: nontemporal loads. The 16-byte stores of a lane lie 32 or
// 64 bytes apart, which the cache merges into whole lines: plain stores (nontemporal ones reached memory as parts of
// lines, FP8 to FP32 at 16 codes a thread 1.6 TB/s against 4.4 at 8).
template <int KIND, int E>
__global__ __launch_bounds__(256) void read_rows_kernel(ReadArgs a) {
    static_assert(E == 8 || (E == 16 && KIND != 0), "16 bytes a load");
    const int which = blockIdx.y;
    const int chunks = a.dim[which] / E;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t per_row = (int64_t)a.hkv * chunks;
    if (chunks == 0 || idx >= a.n * per_row) return;
    const int64_t i = idx / per_row;
    const int rest = (int)(idx - i * per_row);
    const int h = rest / chunks, c = rest - h * chunks;
    int64_t slot;
    if (a.slots) {
        slot = a.slots[i];
    } else {
        const int64_t entry = i / a.page;
        slot = (a.table ? (int64_t)a.table[entry] : a.table64[entry]) * a.page + i % a.page;
    }
    float x[E];
    u32x4 as_stored = {0u, 0u, 0u, 0u};      // 16-bit pages read back in their own type: the bits as they are
    if (slot < 0 || (a.pool_slots > 0 && slot >= a.pool_slots)) {
#pragma unroll
        for (int j = 0; j < E; ++j) x[j] = 0.0f;
    } else {
        const int64_t row = slot * a.hkv + h;
        if constexpr (KIND == 0) {
            const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a.pages[which] + (row * a.dim[which] + c * 8) * 2));
            const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
            as_stored = w;
            if (a.f16_pages) {
#pragma unroll
                for (int j = 0; j < 4; ++j) x[2 * j] = f16_lo(ws[j]), x[2 * j + 1] = f16_hi(ws[j]);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) x[2 * j] = bf16_lo(ws[j]), x[2 * j + 1] = bf16_hi(ws[j]);
            }
        } else {
            uint32_t ws[E / 4];
            const uint8_t* src = a.pages[which] + row * a.dim[which] + c * E;
            if constexpr (E == 16) {
                const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src));
                ws[0] = w.x, ws[1] = w.y, ws[2] = w.z, ws[3] = w.w;
            } else {
                const u32x2 w = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(src));
                ws[0] = w.x, ws[1] = w.y;
            }
            if constexpr (KIND == 3) {
#pragma unroll
                for (int j = 0; j < E; ++j) x[j] = (float)(int8_t)(ws[j >> 2] >> (8 * (j & 3)));
            } else {
#pragma unroll
                for (int j = 0; j < E / 4; ++j) {
                    const f32x2 lo = e4m3_pair<false>(ws[j]), hi = e4m3_pair<true>(ws[j]);
                    x[4 * j] = lo.x, x[4 * j + 1] = lo.y, x[4 * j + 2] = hi.x, x[4 * j + 3] = hi.y;
                }
            }
            const float s = KIND == 1 ? (a.head_mult ? a.head_mult[which * a.hkv + h] : a.mult[which]) : a.scales[which][row];
#pragma unroll
            for (int j = 0; j < E; ++j) x[j] = x[j] * s;
        }
    }
    const int64_t at = (i * a.hkv + h) * a.dim[which] + c * E;
    if (a.out_dtype == CRIT_PKV_F32) {
        u32x4* o = reinterpret_cast<u32x4*>(reinterpret_cast<float*>(a.out[which]) + at);
#pragma unroll
        for (int j = 0; j < E / 4; ++j) {
            const u32x4 w = {f2u(x[4 * j]), f2u(x[4 * j + 1]), f2u(x[4 * j + 2]), f2u(x[4 * j + 3])};
            o[j] = w;
        }
    } else {
        u32x4* o = reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(a.out[which]) + at);
        const bool bf = a.out_dtype == CRIT_PKV_BF16;
        if constexpr (KIND == 0) {
            // (the reference's .to(compute) of the pages' own dtype is the tensor itself: a NaN keeps its payload)
            if (bf != (a.f16_pages != 0)) {
                o[0] = as_stored;
                return;
            }
        }
#pragma unroll
        for (int j = 0; j < E / 8; ++j) {
            u32x4 w;
            w.x = bf ? pack_bf16(x[8 * j], x[8 * j + 1]) : pack_f16(x[8 * j], x[8 * j + 1]);
            w.y = bf ? pack_bf16(x[8 * j + 2], x[8 * j + 3]) : pack_f16(x[8 * j + 2], x[8 * j + 3]);
            w.z = bf ? pack_bf16(x[8 * j + 4], x[8 * j + 5]) : pack_f16(x[8 * j + 4], x[8 * j + 5]);
            w.w = bf ? pack_bf16(x[8 * j + 6], x[8 * j + 7]) : pack_f16(x[8 * j + 6], x[8 * j + 7]);
            o[j] = w;
        }
    }
}

}   // namespace

int launch_read_rows(const crit_pkv_read_params* p, hipStream_t stream) {
    if (!p) return CRIT_PKV_E_NULL;
    if (p->n == 0) return 0;
    if (!p->key_pages || !p->out_keys) return CRIT_PKV_E_NULL;
    if ((p->value_pages == nullptr) != (p->out_values == nullptr)) return CRIT_PKV_E_NULL;
    const int sources = (p->slots != nullptr) + (p->table != nullptr) + (p->table64 != nullptr);
    if (sources != 1) return CRIT_PKV_E_NULL;
    const int dv = p->value_pages ? p->value_dim : 0;
    if (p->n < 0 || p->pool_slots < 0 || p->kv_heads < 1 || p->head_dim < 8 || p->head_dim % 8 || dv % 8 || (p->value_pages && dv < 8) ||
        (!p->slots && p->page < 1))
        return CRIT_PKV_E_GEOMETRY;
    if (p->kind < 0 || p->kind > 3 || p->out_dtype < 0 || p->out_dtype > 2) return CRIT_PKV_E_DTYPE;
    if (p->kind == CRIT_PKV_KIND_16BIT && p->page_dtype != CRIT_PKV_BF16 && p->page_dtype != CRIT_PKV_F16) return CRIT_PKV_E_DTYPE;
    if (p->kind >= CRIT_PKV_KIND_FP8_ROW && (!p->key_scales || (p->value_pages && !p->value_scales))) return CRIT_PKV_E_NULL;
    const uintptr_t align = reinterpret_cast<uintptr_t>(p->key_pages) | reinterpret_cast<uintptr_t>(p->value_pages) |
                            reinterpret_cast<uintptr_t>(p->out_keys) | reinterpret_cast<uintptr_t>(p->out_values);
    if (align % 16) return CRIT_PKV_E_GEOMETRY;
    ReadArgs a;
    a.pages[0] = reinterpret_cast<const uint8_t*>(p->key_pages), a.pages[1] = reinterpret_cast<const uint8_t*>(p->value_pages);
    a.scales[0] = p->key_scales, a.scales[1] = p->value_scales;
    a.head_mult = p->head_multipliers, a.mult[0] = p->key_multiplier, a.mult[1] = p->value_multiplier;
    a.out[0] = p->out_keys, a.out[1] = p->out_values;
    a.slots = p->slots, a.table = p->table, a.table64 = p->table64, a.n = p->n, a.pool_slots = p->pool_slots;
    a.hkv = p->kv_heads, a.dim[0] = p->head_dim, a.dim[1] = dv, a.page = p->page, a.kind = p->kind;
    a.f16_pages = p->page_dtype == CRIT_PKV_F16, a.out_dtype = p->out_dtype;
    const int widest = p->head_dim > dv ? p->head_dim : dv;
    const bool wide = p->kind != 0 && p->head_dim % 16 == 0 && dv % 16 == 0 && p->out_dtype != CRIT_PKV_F32;
    const int64_t threads = p->n * p->kv_heads * (widest / (wide ? 16 : 8));
    const int64_t blocks = (threads + 255) / 256;
    if (blocks > 0x7fffffff) return CRIT_PKV_E_GEOMETRY;
    const dim3 grid((unsigned)blocks, p->value_pages ? 2u : 1u);
    switch (p->kind * 2 + (wide ? 1 : 0)) {
        case 0: hipLaunchKernelGGL((read_rows_kernel<0, 8>), grid, dim3(256), 0, stream, a); break;
        case 2: hipLaunchKernelGGL((read_rows_kernel<1, 8>), grid, dim3(256), 0, stream, a); break;
        case 3: hipLaunchKernelGGL((read_rows_kernel<1, 16>), grid, dim3(256), 0, stream, a); break;
        case 4: hipLaunchKernelGGL((read_rows_kernel<2, 8>), grid, dim3(256), 0, stream, a); break;
        case 5: hipLaunchKernelGGL((read_rows_kernel<2, 16>), grid, dim3(256), 0, stream, a); break;
        case 6: hipLaunchKernelGGL((read_rows_kernel<3, 8>), grid, dim3(256), 0, stream, a); break;
        default: hipLaunchKernelGGL((read_rows_kernel<3, 16>), grid, dim3(256), 0, stream, a); break;
    }
    return (int)hipGetLastError();
}

}   // namespace pkv
