// The C ABI: argument checks live in the launchers; this file only forwards and names errors.
#include "pkv_launch.hpp"

extern "C" {

int crit_pkv_write(const crit_pkv_write_params* p, void* stream) {
    return pkv::launch_write(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_attend(const crit_pkv_attend_params* p, void* stream) {
    return pkv::launch_attend(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_attend_static(const crit_pkv_attend_params* p, void* stream) {
    return pkv::launch_attend_static(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_merge(const crit_pkv_merge_params* p, void* stream) {
    return pkv::launch_merge(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_prefill(const crit_pkv_prefill_params* p, void* stream) {
    return pkv::launch_prefill(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_slots_at(const crit_pkv_slots_params* p, void* stream) {
    return pkv::launch_slots_at(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_compact(const crit_pkv_compact_params* p, void* stream) {
    return pkv::launch_compact(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_copy_pages(const crit_pkv_copy_pages_params* p, void* stream) {
    return pkv::launch_copy_pages(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_latent_attend(const crit_pkv_latent_params* p, void* stream) {
    return pkv::launch_latent(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_latent_write(const crit_pkv_latent_write_params* p, void* stream) {
    return pkv::launch_latent_write(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_index_scores(const crit_pkv_index_scores_params* p, void* stream) {
    return pkv::launch_index_scores(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_index_topk(const crit_pkv_index_topk_params* p, void* stream) {
    return pkv::launch_index_topk(p, reinterpret_cast<hipStream_t>(stream));
}

int64_t crit_pkv_index_topk_work_bytes(int32_t tokens, int32_t n, int32_t k) { return pkv::index_topk_work_bytes(tokens, n, k); }

int crit_pkv_round(const crit_pkv_round_params* p, void* stream) {
    return pkv::launch_round(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_step_buffers(const crit_pkv_step_params* p, void* stream) {
    return pkv::launch_step_buffers(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_read_rows(const crit_pkv_read_params* p, void* stream) {
    return pkv::launch_read_rows(p, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_stream_read(const void* data, int64_t bytes, float* sink, void* stream) {
    return pkv::launch_stream_read(data, bytes, sink, reinterpret_cast<hipStream_t>(stream));
}

int crit_pkv_stream_capture(void* stream, unsigned long long* id) {
    if (!id) return CRIT_PKV_E_NULL;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long found = 0;
    const hipError_t e = hipStreamGetCaptureInfo(reinterpret_cast<hipStream_t>(stream), &status, &found);
    if (e != hipSuccess) return (int)e;
    *id = status == hipStreamCaptureStatusActive ? (found ? found : ~0ull) : 0;
    return 0;
}

int crit_pkv_abi_version(void) { return CRIT_PKV_ABI_VERSION; }

int crit_pkv_params_size(int which) {
    switch (which) {
        case 0: return (int)sizeof(crit_pkv_write_params);
        case 1: return (int)sizeof(crit_pkv_attend_params);
        case 2: return (int)sizeof(crit_pkv_merge_params);
        case 3: return (int)sizeof(crit_pkv_prefill_params);
        case 4: return (int)sizeof(crit_pkv_slots_params);
        case 5: return (int)sizeof(crit_pkv_compact_params);
        case 6: return (int)sizeof(crit_pkv_copy_pages_params);
        case 7: return (int)sizeof(crit_pkv_read_params);
        case 8: return (int)sizeof(crit_pkv_round_params);
        case 9: return (int)sizeof(crit_pkv_step_params);
        case 10: return (int)sizeof(crit_pkv_latent_params);
        case 11: return (int)sizeof(crit_pkv_index_scores_params);
        case 12: return (int)sizeof(crit_pkv_index_topk_params);
        case 13: return (int)sizeof(crit_pkv_latent_write_params);
    }
    return -1;
}

const char* crit_pkv_error(int code) {
    switch (code) {
        case 0: return "ok";
        case CRIT_PKV_E_GEOMETRY: return "crit_pkv: a shape the kernels do not take (head dims 16 to 256 in powers of two (prompt chunks: 64 or 128, keys and values of one width), query heads a multiple of the KV heads, 1..64 columns, 16-byte aligned rows; pool stores in multiples of 4 bytes, tree paths of up to 256 columns)";
        case CRIT_PKV_E_DTYPE: return "crit_pkv: a dtype or page kind the kernels do not take";
        case CRIT_PKV_E_NULL: return "crit_pkv: a required pointer is NULL";
        case CRIT_PKV_E_WORKSPACE: return "crit_pkv: partitions, piece or the partial arrays do not fit the launch";
    }
    if (code == CRIT_PKV_E_SCRATCH) return "crit_pkv: the launch's partials (rows x columns x heads x partitions x (value_dim + 2) floats) do not fit the library's static scratch (CRIT_PKV_STATIC_SCRATCH_BYTES), or its address could not be had: use crit_pkv_attend with a workspace";
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "crit_pkv: unknown error";
}

}   // extern "C"
