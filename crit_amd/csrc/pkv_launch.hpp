// Host-side launchers, one per translation unit of kernels; the C ABI (pkv_abi.hip) forwards to them.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/crit_pkv.h"

namespace pkv {
int launch_write(const crit_pkv_write_params* p, hipStream_t stream);
int launch_attend(const crit_pkv_attend_params* p, hipStream_t stream);
int launch_attend_static(const crit_pkv_attend_params* p, hipStream_t stream);
int launch_merge(const crit_pkv_merge_params* p, hipStream_t stream);
int launch_prefill(const crit_pkv_prefill_params* p, hipStream_t stream);
int launch_slots_at(const crit_pkv_slots_params* p, hipStream_t stream);
int launch_compact(const crit_pkv_compact_params* p, hipStream_t stream);
int launch_copy_pages(const crit_pkv_copy_pages_params* p, hipStream_t stream);
int launch_round(const crit_pkv_round_params* p, hipStream_t stream);
int launch_step_buffers(const crit_pkv_step_params* p, hipStream_t stream);
int launch_latent(const crit_pkv_latent_params* p, hipStream_t stream);
int launch_latent_write(const crit_pkv_latent_write_params* p, hipStream_t stream);
int launch_index_scores(const crit_pkv_index_scores_params* p, hipStream_t stream);
int launch_index_topk(const crit_pkv_index_topk_params* p, hipStream_t stream);
int64_t index_topk_work_bytes(int tokens, int n, int k);
int launch_read_rows(const crit_pkv_read_params* p, hipStream_t stream);
int launch_stream_read(const void* data, int64_t bytes, float* sink, hipStream_t stream);
// Compute units of the current device (cached per device), or 0 if the query fails.
int compute_units();
}   // namespace pkv
