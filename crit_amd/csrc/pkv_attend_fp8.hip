// Split / fused decode kernels over fp8 pages (one page kind per translation unit: they compile in parallel).
#include "pkv_attend_inst.hpp"
#include "pkv_launch.hpp"

namespace pkv {
int launch_attend_fp8(const AttendArgs& a, int lpr, int qr, bool fused, bool page16, dim3 grid, hipStream_t stream) {
    return launch_kind_impl<1, false>(a, lpr, qr, fused, page16, grid, stream);
}
}   // namespace pkv
