"""ctypes mirror of include/crit_pkv.h and the loader of libcrit_pkv.so.

The library is looked for at $CRIT_PKV_LIB, beside this package (a staged copy inside a crit kernel cache) and in
crit_amd/lib (the in-tree build). If none exists and hipcc is on PATH it is built once, in-tree; otherwise loading
fails: there is no other implementation behind this module.
"""
import ctypes
import os
import shutil

_HERE = os.path.dirname(os.path.abspath(__file__))
NAME = "libcrit_pkv.so"
ABI_VERSION = 20

KIND_16BIT, KIND_FP8, KIND_FP8_ROW, KIND_INT8 = 0, 1, 2, 3
F32, BF16, F16 = 0, 1, 2

_p, _i64, _i32, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_float


class WriteParams(ctypes.Structure):
    _fields_ = [("keys", _p), ("values", _p), ("slots", _p), ("key_pages", _p), ("value_pages", _p),
                ("key_scales", _p), ("value_scales", _p), ("head_multipliers", _p),
                ("tokens", _i64), ("key_stride_t", _i64), ("key_stride_h", _i64), ("value_stride_t", _i64),
                ("value_stride_h", _i64),
                ("kv_heads", _i32), ("head_dim", _i32), ("value_dim", _i32), ("kind", _i32), ("page_dtype", _i32),
                ("in_dtype", _i32), ("key_multiplier", _f32), ("value_multiplier", _f32),
                ("rope_table", _p), ("rope_positions", _p), ("rope_rows", _i64), ("rope_interleaved", _i32),
                ("rope_scale", _f32), ("norm_weight", _p), ("norm_eps", _f32), ("norm_offset", _f32)]


class AttendParams(ctypes.Structure):
    _fields_ = [("q", _p), ("key_pages", _p), ("value_pages", _p), ("key_scales", _p), ("value_scales", _p),
                ("head_multipliers", _p), ("tables", _p), ("rows", _p), ("starts", _p), ("counts", _p), ("firsts", _p),
                ("offsets", _p), ("partial_out", _p), ("partial_max", _p), ("partial_sum", _p), ("out", _p),
                ("lse", _p), ("sinks", _p), ("parents", _p), ("parents64", _p), ("blocks", _p),
                ("q_stride_t", _i64), ("q_stride_h", _i64), ("out_stride_t", _i64), ("out_stride_h", _i64),
                ("table_stride", _i64), ("blocks_stride", _i64),
                ("table_width", _i32), ("n_rows", _i32), ("columns", _i32), ("heads", _i32), ("kv_heads", _i32),
                ("head_dim", _i32), ("value_dim", _i32), ("page", _i32), ("kind", _i32), ("page_dtype", _i32),
                ("out_dtype", _i32), ("partitions", _i32), ("piece", _i32), ("fused", _i32), ("sliding", _i32), ("phases", _i32),
                ("blocks_k", _i32), ("block_size", _i32),
                ("scale", _f32), ("key_multiplier", _f32), ("value_multiplier", _f32),
                ("fresh_keys", _p), ("fresh_values", _p), ("fresh_shifts", _p), ("fresh_firsts", _p),
                ("fresh_stride_k", _i64), ("fresh_stride_v", _i64), ("fresh_rows", _i64), ("fresh_per_row", _i32),
                ("rows_are_64", _i32), ("launch_state", _p),
                ("derive_table", _p), ("derive_eps", _f32), ("derive_rot", _i32), ("derive_weighted", _i32),
                ("int8_qk", _i32)]


class MergeParams(ctypes.Structure):
    _fields_ = [("outs", _p), ("lses", _p), ("out", _p), ("lse", _p), ("rows", _i64), ("parts", _i32),
                ("value_dim", _i32), ("in_dtype", _i32)]


class PrefillParams(ctypes.Structure):
    _fields_ = [("q", _p), ("key_pages", _p), ("value_pages", _p), ("key_scales", _p), ("value_scales", _p),
                ("head_multipliers", _p), ("tables", _p), ("tables64", _p), ("table_rows", _p), ("starts", _p),
                ("counts", _p), ("positions", _p), ("out", _p), ("lse", _p), ("sinks", _p),
                ("q_stride_t", _i64), ("q_stride_h", _i64), ("out_stride_t", _i64), ("out_stride_h", _i64),
                ("table_stride", _i64),
                ("table_width", _i32), ("chunks", _i32), ("max_count", _i32), ("heads", _i32), ("kv_heads", _i32),
                ("head_dim", _i32), ("page", _i32), ("kind", _i32), ("page_dtype", _i32), ("out_dtype", _i32),
                ("sliding", _i32), ("scale", _f32), ("key_multiplier", _f32), ("value_multiplier", _f32),
                ("fresh_keys", _p), ("fresh_values", _p), ("fresh_firsts", _p), ("fresh_state", _p),
                ("fresh_stride_k", _i64), ("fresh_stride_v", _i64), ("int8_qk", _i32)]


class Store(ctypes.Structure):
    _fields_ = [("base", _p), ("layer_stride", _i64), ("row_bytes", _i64)]


MAX_STORES, MAX_PATH = 4, 256


class SlotsParams(ctypes.Structure):
    _fields_ = [("round_tables", _p), ("round_capacity", _p), ("slots", _p), ("rows", _p), ("positions", _p), ("out", _p),
                ("n", _i64), ("round_slots", _i64), ("table_stride", _i64), ("n_slots", _i64),
                ("table_pages", _i32), ("page", _i32), ("dump", _i32)]


class CompactParams(ctypes.Structure):
    _fields_ = [("round_tables", _p), ("round_capacity", _p), ("start", _p), ("emitted", _p), ("path", _p), ("moved", _p),
                ("stores", Store * MAX_STORES),
                ("rows", _i64), ("round_slots", _i64), ("table_stride", _i64), ("path_stride", _i64),
                ("n_stores", _i32), ("layers", _i32), ("width", _i32), ("path_is_32", _i32), ("table_pages", _i32),
                ("page", _i32), ("dump", _i32)]


class CopyPagesParams(ctypes.Structure):
    _fields_ = [("source", _p), ("target", _p), ("stores", Store * MAX_STORES), ("n", _i64), ("pool_pages", _i64),
                ("n_stores", _i32), ("layers", _i32), ("page", _i32)]


class RoundParams(ctypes.Structure):
    _fields_ = [("round_lengths", _p), ("start", _p), ("moved", _p), ("emitted", _p), ("frontier", _p), ("rows", _i64),
                ("commit", _i32)]


class StepParams(ctypes.Structure):
    _fields_ = [("round_tables", _p), ("round_capacity", _p), ("round_lengths", _p), ("slot", _p), ("counts", _p),
                ("firsts", _p), ("d_slots", _p), ("positions_t", _p), ("rows_t", _p), ("starts_t", _p), ("d_rows", _p),
                ("d_starts", _p), ("d_counts", _p), ("d_firsts", _p), ("d_offsets", _p), ("d_tables", _p), ("totals", _p),
                ("rows", _i64), ("round_slots", _i64), ("table_stride", _i64), ("d_tables_stride", _i64),
                ("step_tokens", _i64), ("step_rows", _i64), ("count_each", _i64), ("window", _i64),
                ("table_pages", _i32), ("page", _i32), ("dump", _i32)]


class LatentParams(ctypes.Structure):
    _fields_ = [("q", _p), ("cache", _p), ("scales", _p), ("tables", _p), ("rows", _p), ("starts", _p), ("counts", _p),
                ("firsts", _p), ("partial_out", _p), ("partial_max", _p), ("partial_sum", _p), ("out", _p), ("lse", _p),
                ("sinks", _p),
                ("q_stride_t", _i64), ("q_stride_h", _i64), ("out_stride_t", _i64), ("out_stride_h", _i64), ("table_stride", _i64),
                ("table_width", _i32), ("n_rows", _i32), ("columns", _i32), ("heads", _i32), ("rank", _i32), ("rope", _i32),
                ("page", _i32), ("cache_dtype", _i32), ("q_dtype", _i32), ("out_dtype", _i32), ("scales_per_row", _i32),
                ("partitions", _i32), ("piece", _i32), ("rows_are_64", _i32), ("phases", _i32), ("tile_rows", _i32),
                ("scale", _f32)]


class LatentWriteParams(ctypes.Structure):
    _fields_ = [("latent", _p), ("rope", _p), ("slots", _p), ("cache", _p), ("scales", _p),
                ("tokens", _i64), ("latent_stride", _i64), ("rope_stride", _i64),
                ("rank", _i32), ("rope_width", _i32), ("in_dtype", _i32), ("cache_dtype", _i32)]


class IndexScoresParams(ctypes.Structure):
    _fields_ = [("q", _p), ("keys", _p), ("key_scales", _p), ("weights", _p), ("ends", _p), ("slots", _p), ("out", _p),
                ("q_stride_t", _i64), ("q_stride_h", _i64), ("key_stride", _i64), ("weights_stride", _i64),
                ("out_stride", _i64), ("slots_stride", _i64),
                ("tokens", _i32), ("n", _i32), ("group", _i32), ("heads", _i32), ("dim", _i32), ("key_dtype", _i32),
                ("q_dtype", _i32), ("slots_are_64", _i32), ("scale", _f32)]


class IndexTopkParams(ctypes.Structure):
    _fields_ = [("scores", _p), ("ends", _p), ("out", _p), ("work", _p), ("scores_stride", _i64), ("out_stride", _i64),
                ("work_bytes", _i64), ("tokens", _i32), ("n", _i32), ("k", _i32)]


class ReadParams(ctypes.Structure):
    _fields_ = [("key_pages", _p), ("value_pages", _p), ("key_scales", _p), ("value_scales", _p), ("head_multipliers", _p),
                ("slots", _p), ("table", _p), ("table64", _p), ("out_keys", _p), ("out_values", _p), ("n", _i64), ("pool_slots", _i64),
                ("kv_heads", _i32), ("head_dim", _i32), ("value_dim", _i32), ("page", _i32), ("kind", _i32),
                ("page_dtype", _i32), ("out_dtype", _i32), ("key_multiplier", _f32), ("value_multiplier", _f32)]


STATIC_SCRATCH_BYTES = 32 << 20

SYMBOLS = ("crit_pkv_write", "crit_pkv_attend", "crit_pkv_attend_static", "crit_pkv_merge", "crit_pkv_prefill", "crit_pkv_slots_at",
           "crit_pkv_compact", "crit_pkv_copy_pages", "crit_pkv_round", "crit_pkv_step_buffers", "crit_pkv_latent_attend", "crit_pkv_latent_write", "crit_pkv_index_scores", "crit_pkv_index_topk", "crit_pkv_index_topk_work_bytes", "crit_pkv_read_rows", "crit_pkv_abi_version", "crit_pkv_params_size", "crit_pkv_error",
           "crit_pkv_stream_read", "crit_pkv_stream_capture")

_lib = None


def candidates():
    found = []
    if os.environ.get("CRIT_PKV_LIB"):
        found.append(os.environ["CRIT_PKV_LIB"])
    found.append(os.path.join(_HERE, NAME))
    found.append(os.path.join(os.path.dirname(_HERE), "lib", NAME))
    return found


def _build_in_tree():
    """The in-tree build (crit_amd/build.py), when this package sits inside crit_amd and hipcc exists."""
    script = os.path.join(os.path.dirname(_HERE), "build.py")
    if not os.path.exists(script) or shutil.which("hipcc") is None:
        return None
    import importlib.util
    spec = importlib.util.spec_from_file_location("_crit_pkv_build", script)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module.build(verbose=False)


def load():
    """The loaded library (a ctypes.CDLL with typed entry points); raises RuntimeError when it cannot be had."""
    global _lib
    if _lib is not None:
        return _lib
    path = next((c for c in candidates() if os.path.exists(c)), None)
    if path is None:
        path = _build_in_tree()
    if path is None:
        raise RuntimeError(f"{NAME} is not built (looked in {', '.join(candidates())}) and hipcc is not available: "
                           "run `python -m crit_amd.build`; this module has no other implementation")
    lib = ctypes.CDLL(path)
    for name in SYMBOLS:
        if not hasattr(lib, name):
            raise RuntimeError(f"{path} does not export {name}")
    lib.crit_pkv_error.restype = ctypes.c_char_p
    lib.crit_pkv_error.argtypes = [ctypes.c_int]
    lib.crit_pkv_params_size.argtypes = [ctypes.c_int]
    for name, struct in (("crit_pkv_write", WriteParams), ("crit_pkv_attend", AttendParams),
                         ("crit_pkv_attend_static", AttendParams),
                         ("crit_pkv_merge", MergeParams), ("crit_pkv_prefill", PrefillParams),
                         ("crit_pkv_slots_at", SlotsParams), ("crit_pkv_compact", CompactParams),
                         ("crit_pkv_copy_pages", CopyPagesParams), ("crit_pkv_round", RoundParams),
                         ("crit_pkv_step_buffers", StepParams), ("crit_pkv_latent_attend", LatentParams),
                         ("crit_pkv_latent_write", LatentWriteParams),
                         ("crit_pkv_index_scores", IndexScoresParams), ("crit_pkv_index_topk", IndexTopkParams),
                         ("crit_pkv_read_rows", ReadParams)):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.POINTER(struct), ctypes.c_void_p]
    lib.crit_pkv_index_topk_work_bytes.restype = ctypes.c_int64
    lib.crit_pkv_index_topk_work_bytes.argtypes = [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32]
    lib.crit_pkv_stream_capture.restype = ctypes.c_int
    lib.crit_pkv_stream_capture.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_ulonglong)]
    lib.crit_pkv_stream_read.restype = ctypes.c_int
    lib.crit_pkv_stream_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
    if lib.crit_pkv_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{path} speaks ABI {lib.crit_pkv_abi_version()}, this package {ABI_VERSION}: rebuild it")
    for which, struct in enumerate((WriteParams, AttendParams, MergeParams, PrefillParams, SlotsParams, CompactParams,
                                    CopyPagesParams, ReadParams, RoundParams, StepParams, LatentParams,
                                    IndexScoresParams, IndexTopkParams, LatentWriteParams)):
        if lib.crit_pkv_params_size(which) != ctypes.sizeof(struct):
            raise RuntimeError(f"{path}: parameter struct {which} is {lib.crit_pkv_params_size(which)} bytes, the "
                               f"Python mirror {ctypes.sizeof(struct)}: rebuild the library")
    lib.path = path
    _lib = lib
    return lib


def capture_id(stream):
    """The id of the capture `stream` (a handle) is recording into, 0 when it is not capturing. The cell the library
    writes the id into is the call's own: ctypes lets other threads run during the call, and each owner launches from
    its own thread."""
    cell = ctypes.c_ulonglong()
    code = load().crit_pkv_stream_capture(stream, ctypes.byref(cell))
    if code:
        check(code, "crit_pkv_stream_capture")
    return cell.value


def check(code, what):
    """Raise for a non-zero return of an entry point: ValueError for a refused launch, RuntimeError for a HIP error."""
    if code == 0:
        return
    text = load().crit_pkv_error(code).decode()
    if code < 0:
        raise ValueError(f"{what}: {text}")
    raise RuntimeError(f"{what}: HIP error {code}: {text}")
