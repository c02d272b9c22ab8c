// Launch of the split (or fused) kernels for ONE page kind; each pkv_attend_k*.hip instantiates one kind so the
// kinds compile in parallel.
#pragma once
#include "pkv_attend_mfma.hpp"
#include "pkv_attend128.hpp"
#include "pkv_attend_generic.hpp"
#include "pkv_launch.hpp"

namespace pkv {

template <int KIND, bool F16, int QR, bool FUSED>
static int launch_one(const AttendArgs& a, int lpr, bool page16, dim3 grid, hipStream_t stream) {
    // (which tile heights each variant is built for: launch_attend picks among them)
    constexpr bool LISTS = QR == 1 || QR == 4, SPECIAL = QR == 2 || QR == 8;
    if (a.blocks && (FUSED || !LISTS)) return CRIT_PKV_E_GEOMETRY;
    if ((a.derive_table || a.fv) && !SPECIAL) return CRIT_PKV_E_GEOMETRY;
    if constexpr (!FUSED && LISTS) {
        if (a.blocks && a.fast128) {
            // block lists whose steps lie in one block and one page: the bandwidth path walking each column's list
            AttendArgs u = a;
            u.units_x = (int)grid.x, u.units_y = (int)grid.y + kTailClasses - 1;
            const int64_t units = (int64_t)u.units_x * u.units_y;
            if (units > 0x7fffffff) return CRIT_PKV_E_GEOMETRY;
            const int64_t resident = (int64_t)compute_units() * attend_waves(KIND, QR);
            const dim3 pgrid((unsigned)(units < resident ? units : resident));
            if (units <= resident) u.ticket = nullptr;      // (a unit a workgroup: nothing to draw, no counter touched)
            switch (a.heads_per_wave) {
                case 1: hipLaunchKernelGGL((attend128_kernel<KIND, F16, QR, 1, false, true>), pgrid, dim3(256), 0, stream, u); break;
                case 2: hipLaunchKernelGGL((attend128_kernel<KIND, F16, QR, 2, false, true>), pgrid, dim3(256), 0, stream, u); break;
                default: return CRIT_PKV_E_GEOMETRY;
            }
            return hip_code(hipGetLastError());
        }
        if (a.blocks) {      // other block lists: the generic kernel, each position looked up on its own
            switch (lpr) {
                case 2: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 2, QR, false, true>), grid, dim3(256), 0, stream, a); break;
                case 4: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 4, QR, false, true>), grid, dim3(256), 0, stream, a); break;
                case 8: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 8, QR, false, true>), grid, dim3(256), 0, stream, a); break;
                case 16: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 16, QR, false, true>), grid, dim3(256), 0, stream, a); break;
                case 32: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 32, QR, false, true>), grid, dim3(256), 0, stream, a); break;
                default: return CRIT_PKV_E_GEOMETRY;
            }
            return hip_code(hipGetLastError());
        }
    }
    if constexpr (SPECIAL && KIND == 3 && FUSED) {
        if (a.iqk) {      // INT8 queries against INT8 keys: a prompt chunk's window rows (with or without its own fresh rows)
            switch (a.fv ? lpr : -lpr) {
#define PKV_IQK(L) \
    case L: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, L, QR, true, false, true, false, true>), grid, dim3(256), 0, stream, a); break; \
    case -L: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, L, QR, true, false, false, false, true>), grid, dim3(256), 0, stream, a); break;
                PKV_IQK(2) PKV_IQK(4) PKV_IQK(8) PKV_IQK(16) PKV_IQK(32)
#undef PKV_IQK
                default: return CRIT_PKV_E_GEOMETRY;
            }
            return hip_code(hipGetLastError());
        }
    }
    if (a.iqk) return CRIT_PKV_E_GEOMETRY;
    if constexpr (SPECIAL) {
    if (a.derive_table && a.fv) {      // derived keys over pages and fresh value rows
        switch (lpr) {
            case 2: if constexpr (QR == 8) { hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 2, QR, FUSED, false, true, true>), grid, dim3(256), 0, stream, a); break; } return CRIT_PKV_E_GEOMETRY;
            case 4: if constexpr (QR == 8) { hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 4, QR, FUSED, false, true, true>), grid, dim3(256), 0, stream, a); break; } return CRIT_PKV_E_GEOMETRY;
            case 8: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 8, QR, FUSED, false, true, true>), grid, dim3(256), 0, stream, a); break;
            case 16: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 16, QR, FUSED, false, true, true>), grid, dim3(256), 0, stream, a); break;
            case 32: if constexpr (QR == 8) { hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 32, QR, FUSED, false, true, true>), grid, dim3(256), 0, stream, a); break; } return CRIT_PKV_E_GEOMETRY;
            default: return CRIT_PKV_E_GEOMETRY;
        }
    } else if (a.derive_table) {      // keys derived from the value rows: the generic kernel's variant (any head width; the widths other than 64 and 128 in tiles of 8 rows only)
        switch (lpr) {
            case 2: if constexpr (QR == 8) { hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 2, QR, FUSED, false, false, true>), grid, dim3(256), 0, stream, a); break; } return CRIT_PKV_E_GEOMETRY;
            case 4: if constexpr (QR == 8) { hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 4, QR, FUSED, false, false, true>), grid, dim3(256), 0, stream, a); break; } return CRIT_PKV_E_GEOMETRY;
            case 8: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 8, QR, FUSED, false, false, true>), grid, dim3(256), 0, stream, a); break;
            case 16: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 16, QR, FUSED, false, false, true>), grid, dim3(256), 0, stream, a); break;
            case 32: if constexpr (QR == 8) { hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 32, QR, FUSED, false, false, true>), grid, dim3(256), 0, stream, a); break; } return CRIT_PKV_E_GEOMETRY;
            default: return CRIT_PKV_E_GEOMETRY;
        }
    } else if (a.fv) {       // fresh rows beside the pages: the generic kernel's variant that reads both (any head width; the widths other than 64 and 128 in tiles of 8 rows only)
        switch (lpr) {
            case 2: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 2, QR, FUSED, false, true>), grid, dim3(256), 0, stream, a); break;
            case 4: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 4, QR, FUSED, false, true>), grid, dim3(256), 0, stream, a); break;
            case 8: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 8, QR, FUSED, false, true>), grid, dim3(256), 0, stream, a); break;
            case 16: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 16, QR, FUSED, false, true>), grid, dim3(256), 0, stream, a); break;
            case 32: hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 32, QR, FUSED, false, true>), grid, dim3(256), 0, stream, a); break;
            default: return CRIT_PKV_E_GEOMETRY;
        }
    }
    if (a.derive_table || a.fv) return hip_code(hipGetLastError());
    }
    if (lpr == 16) {
        hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 16, QR, FUSED>), grid, dim3(256), 0, stream, a);
    } else if (lpr == 8) {
        hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 8, QR, FUSED>), grid, dim3(256), 0, stream, a);
    } else if (lpr == 32) {
        hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 32, QR, FUSED>), grid, dim3(256), 0, stream, a);
    } else if (lpr == 4) {
        hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 4, QR, FUSED>), grid, dim3(256), 0, stream, a);
    } else if (lpr == 2) {
        hipLaunchKernelGGL((attend_generic_kernel<KIND, F16, 2, QR, FUSED>), grid, dim3(256), 0, stream, a);
    } else {
        return CRIT_PKV_E_GEOMETRY;
    }
    return hip_code(hipGetLastError());
}

// 128- and 256-wide heads over pages of a multiple of 16 positions: the bandwidth path, resident workgroups pulling units.
template <int KIND, bool F16>
static int launch_mfma(const AttendArgs& a, bool fused, dim3 grid, hipStream_t stream) {
    AttendArgs u = a;
    // (a split launch lists a row's last partition once more for each size class it may fall in)
    u.units_x = (int)grid.x, u.units_y = fused ? (int)grid.y : (int)grid.y + kTailClasses - 1;
    const int64_t units = (int64_t)u.units_x * u.units_y;
    if (units > 0x7fffffff) return CRIT_PKV_E_GEOMETRY;
    const int64_t resident = (int64_t)compute_units() * (a.dk == 256 || a.query_tiles > 2 ? 1 : kMfmaWaves);
    const dim3 pgrid((unsigned)(units < resident ? units : resident));
    // A unit a workgroup at most: nothing to draw, and no counter touched (a draw's round trip and the count of the
    // finished workgroups are a few microseconds at the end of a launch that is one unit long).
    if (units <= resident) u.ticket = nullptr;
    const bool masked = a.parents != nullptr || a.parents64 != nullptr || a.sliding > 0;
    const int which = (a.narrow ? 64 : 0) + (a.dk == 256 ? 8 : (a.heads_per_wave == 2 ? 4 : 0)) + (fused ? 2 : 0) + (masked ? 1 : 0) +
                      (a.query_tiles == 4 ? 12 : (a.query_tiles == 2 ? 24 : 0));
    switch (which) {
#define PKV_MFMA(W, HWV, FU, MA, DH) \
    case W: hipLaunchKernelGGL((attend_mfma_kernel<KIND, F16, HWV, FU, MA, DH>), pgrid, dim3(256), 0, stream, u); break;
        PKV_MFMA(0, 1, false, false, 1) PKV_MFMA(1, 1, false, true, 1) PKV_MFMA(2, 1, true, false, 1) PKV_MFMA(3, 1, true, true, 1)
        PKV_MFMA(4, 2, false, false, 1) PKV_MFMA(5, 2, false, true, 1) PKV_MFMA(6, 2, true, false, 1) PKV_MFMA(7, 2, true, true, 1)
        PKV_MFMA(8, 1, false, false, 2) PKV_MFMA(9, 1, false, true, 2) PKV_MFMA(10, 1, true, false, 2) PKV_MFMA(11, 1, true, true, 2)
#undef PKV_MFMA
        // 64-wide heads in pairs
#define PKV_MFMA_NARROW(W, HWV, FU, MA) \
    case 64 + W: hipLaunchKernelGGL((attend_mfma_kernel<KIND, F16, HWV, FU, MA, 1, 1, true>), pgrid, dim3(256), 0, stream, u); break;
        PKV_MFMA_NARROW(0, 1, false, false) PKV_MFMA_NARROW(1, 1, false, true) PKV_MFMA_NARROW(2, 1, true, false) PKV_MFMA_NARROW(3, 1, true, true)
        PKV_MFMA_NARROW(4, 2, false, false) PKV_MFMA_NARROW(5, 2, false, true) PKV_MFMA_NARROW(6, 2, true, false) PKV_MFMA_NARROW(7, 2, true, true)
#undef PKV_MFMA_NARROW
        // four query tiles a workgroup: split launches of 128-wide heads over 16-bit pages
#define PKV_MFMA_QT(W, HWV, MA) \
    case W:                                                                                                                  \
        if constexpr (KIND == 0) {                                                                                           \
            hipLaunchKernelGGL((attend_mfma_kernel<KIND, F16, HWV, false, MA, 1, 4>), pgrid, dim3(256), 0, stream, u);       \
            break;                                                                                                           \
        }                                                                                                                    \
        return CRIT_PKV_E_GEOMETRY;
        PKV_MFMA_QT(12, 1, false) PKV_MFMA_QT(13, 1, true) PKV_MFMA_QT(16, 2, false) PKV_MFMA_QT(17, 2, true)
#undef PKV_MFMA_QT
        // two query tiles a workgroup, two workgroups a compute unit still
#define PKV_MFMA_QT2(W, HWV, MA) \
    case W:                                                                                                                  \
        if constexpr (KIND <= 3) {                                                                                           \
            hipLaunchKernelGGL((attend_mfma_kernel<KIND, F16, HWV, false, MA, 1, 2>), pgrid, dim3(256), 0, stream, u);       \
            break;                                                                                                           \
        }                                                                                                                    \
        return CRIT_PKV_E_GEOMETRY;
        PKV_MFMA_QT2(24, 1, false) PKV_MFMA_QT2(25, 1, true) PKV_MFMA_QT2(28, 2, false) PKV_MFMA_QT2(29, 2, true)
#undef PKV_MFMA_QT2
        case 32: hipLaunchKernelGGL((attend_mfma_kernel<KIND, F16, 1, false, false, 2, 2>), pgrid, dim3(256), 0, stream, u); break;
        case 33: hipLaunchKernelGGL((attend_mfma_kernel<KIND, F16, 1, false, true, 2, 2>), pgrid, dim3(256), 0, stream, u); break;
        default: return CRIT_PKV_E_GEOMETRY;
    }
    return hip_code(hipGetLastError());
}

template <int KIND, bool F16>
static int launch_kind_impl(const AttendArgs& a, int lpr, int qr, bool fused, bool page16, dim3 grid, hipStream_t stream) {
    if (a.fast128 && !a.blocks) return launch_mfma<KIND, F16>(a, fused, grid, stream);
    switch (qr) {
#define PKV_CASE(Q)                                                                               \
    case Q:                                                                                       \
        return fused ? launch_one<KIND, F16, Q, true>(a, lpr, page16, grid, stream)               \
                     : launch_one<KIND, F16, Q, false>(a, lpr, page16, grid, stream);
        PKV_CASE(1) PKV_CASE(2) PKV_CASE(4) PKV_CASE(8)
#undef PKV_CASE
    }
    return CRIT_PKV_E_GEOMETRY;
}

}   // namespace pkv
