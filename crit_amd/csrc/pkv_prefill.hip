// Chunked prefill over paged KV (placeholder until the MFMA kernel lands).
#include "pkv_common.hpp"
#include "pkv_launch.hpp"

namespace pkv {
int launch_prefill(const crit_pkv_prefill_params* p, hipStream_t stream) {
    (void)p, (void)stream;
    return CRIT_PKV_E_GEOMETRY;
}
}   // namespace pkv
