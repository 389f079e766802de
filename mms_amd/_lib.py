"""ctypes binding of libmmsim.so (the C ABI declared in include/mmsim.h).

The library is looked up next to this package (``mms_amd/libmmsim.so``, built
by ``python -m mms_amd.csrc.build``).  There is no fallback: if the library is
missing, fails to load or finds no gfx950 device, the call raises.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# MMSIM_LIBRARY overrides the location (e.g. to try a differently built library).
LIB_PATH = os.environ.get("MMSIM_LIBRARY") or os.path.join(_HERE, "libmmsim.so")

MMSIM_OK = 0
E_INVALID, E_UNSUPPORTED, E_HIP, E_NOMEM, E_OVERFLOW = -1, -2, -3, -4, -5
STATIC_SCRATCH_BYTES = 32 << 20
BATCHING, WANT_MODEL_COUNTS, WANT_GROUP_COUNTS, WANT_PER_REQUEST, WANT_OP_COUNT = 1, 2, 4, 8, 16

_p_i32 = C.POINTER(C.c_int32)
_p_i64 = C.POINTER(C.c_int64)
_p_f32 = C.POINTER(C.c_float)
_p_f64 = C.POINTER(C.c_double)
_p_u8 = C.POINTER(C.c_uint8)


class MmsimError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"libmmsim error {code}: {message}")
        self.code = code


class Tables(C.Structure):
    _fields_ = [("M", C.c_int32), ("C", C.c_int32), ("Smax", C.c_int32), ("NB", C.c_int32),
                ("cfg_lat", _p_f32), ("cfg_pp", _p_i32), ("batch_sizes", _p_i32),
                ("fixed_overhead", C.c_double)]


class Placements(C.Structure):
    _fields_ = [("B", C.c_int32), ("Gmax", C.c_int32), ("num_groups", _p_i32),
                ("group_cfg", _p_i32), ("gm_off", _p_i64), ("gm_idx", _p_i32)]


class Result(C.Structure):
    _fields_ = [("n_good", _p_i64), ("latency_sum", _p_f64),
                ("model_num_requests", _p_i32), ("model_num_good", _p_i32),
                ("group_num_requests", _p_i32), ("group_num_good", _p_i32),
                ("finish", _p_f64), ("good", _p_u8), ("status", _p_i32), ("fp_ops", _p_i64)]


class Successors(C.Structure):
    _fields_ = [("n", C.c_int32), ("parent", _p_i32), ("group", _p_i32), ("model", _p_i32), ("normalize", C.c_int32)]


class Options(C.Structure):
    """mmsim_options: -1 (switches) / 0 (numbers) leave the choice to the library."""
    _fields_ = [("struct_size", C.c_int32), ("request_loop", C.c_int32), ("waves_per_cu", C.c_int32),
                ("counts_in_lds", C.c_int32), ("tile_order_by_slots", C.c_int32), ("sched_groups", C.c_int32),
                ("segment_requests", C.c_int32), ("sched_spin_limit", C.c_int32), ("skip_ahead", C.c_int32),
                ("xcd_map", C.c_int32), ("batching_lanes", C.c_int32), ("batching_event_slots", C.c_int32),
                ("batching_lds_tables", C.c_int32), ("reserved", C.c_int32), ("stats_scratch_bytes", C.c_int64)]


class DeviceInfo(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("arch", C.c_char * 64), ("compute_units", C.c_int32),
                ("clock_khz", C.c_int32), ("lds_bytes_per_block", C.c_int32), ("hbm_bytes", C.c_int64)]


class ModelStats(C.Structure):
    _fields_ = [("model_num_requests", _p_i32), ("model_num_good", _p_i32),
                ("first_start", _p_f64), ("last_start", _p_f64), ("latency_sum", _p_f64),
                ("latency_mean", _p_f64), ("latency_std", _p_f64), ("latency_p90", _p_f64),
                ("latency_p99", _p_f64)]


class BatchInfo(C.Structure):
    _fields_ = [("lanes", C.c_int32), ("waves", C.c_int32), ("n_seeds", C.c_int32), ("B", C.c_int32),
                ("smax_bucket", C.c_int32), ("max_replicas", C.c_int32), ("slots", C.c_int32),
                ("lds_bytes", C.c_int32), ("requests_total", C.c_int64), ("table_bytes", C.c_int64),
                ("stream_bytes", C.c_int64), ("workgroups", C.c_int32), ("segments", C.c_int32),
                ("launches", C.c_int32), ("waves_per_group", C.c_int32), ("event_slots", C.c_int32),
                ("reserved", C.c_int32)]


# name -> (restype, argtypes); also the list of symbols the header declares
SIGNATURES = {
    "mmsim_abi_version": (C.c_int, []),
    "mmsim_last_error": (C.c_char_p, []),
    "mmsim_ctx_create": (C.c_int, [C.c_int, C.POINTER(C.c_void_p)]),
    "mmsim_ctx_destroy": (None, [C.c_void_p]),
    "mmsim_ctx_device_info": (C.c_int, [C.c_void_p, C.POINTER(DeviceInfo)]),
    "mmsim_options_default": (None, [C.POINTER(Options)]),
    "mmsim_ctx_set_options": (C.c_int, [C.c_void_p, C.POINTER(Options)]),
    "mmsim_batch_create_ex": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_int32, C.POINTER(Tables),
                                         C.POINTER(Placements), C.c_uint32, C.POINTER(Options),
                                         C.POINTER(C.c_void_p)]),
    "mmsim_workload_create": (C.c_int, [C.c_void_p, C.c_int64, C.c_int32, _p_f64, _p_i32, _p_f32,
                                         C.POINTER(C.c_void_p)]),
    "mmsim_workload_destroy": (None, [C.c_void_p]),
    "mmsim_batch_create": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_int32, C.POINTER(Tables),
                                      C.POINTER(Placements), C.c_uint32, C.POINTER(C.c_void_p)]),
    "mmsim_batch_run": (C.c_int, [C.c_void_p]),
    "mmsim_batch_sync": (C.c_int, [C.c_void_p, C.POINTER(C.c_float)]),
    "mmsim_batch_fetch": (C.c_int, [C.c_void_p, C.POINTER(Result)]),
    "mmsim_batch_model_stats": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_int32, C.POINTER(C.c_int64),
                                           C.POINTER(ModelStats)]),
    "mmsim_batch_destroy": (None, [C.c_void_p]),
    "mmsim_batch_get_info": (C.c_int, [C.c_void_p, C.POINTER(BatchInfo)]),
    "mmsim_batch_kernel_name": (C.c_int, [C.c_void_p, C.c_char_p, C.c_size_t]),
    "mmsim_eval_batch": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_int32, C.POINTER(Tables),
                                    C.POINTER(Placements), C.c_uint32, C.POINTER(Result)]),
    "mmsim_eval_successors": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_int32, C.POINTER(Tables),
                                         C.POINTER(Placements), C.POINTER(Successors), C.c_uint32,
                                         C.POINTER(Result)]),
    "mmsim_eval_pairs": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_int32, C.POINTER(Tables),
                                    C.POINTER(Placements), _p_i32, C.c_uint32, C.POINTER(Result)]),
    "mmsim_eval_batch_static": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_int32, C.POINTER(Tables),
                                           C.POINTER(Placements), C.c_uint32, C.POINTER(Result)]),
    "mmsim_simulate_requests_mixed": (C.c_int, [
        C.c_void_p, _p_f64, _p_u8, _p_f64, _p_i32, _p_f32, _p_i32, _p_i32, _p_f32, C.c_int64,
        C.c_int32, C.c_int32, C.c_int32, C.c_double, _p_i32, _p_i32, _p_i32, _p_i32]),
    "mmsim_simulate_requests": (C.c_int, [
        C.c_void_p, _p_f64, _p_u8, _p_f64, _p_i32, _p_f32, _p_i32, _p_f32, _p_f32, C.c_int64,
        C.c_int32, C.c_int32, C.c_double, _p_i32, _p_i32, _p_i32, _p_i32]),
    "mmsim_simulate_requests_mixed_batching": (C.c_int, [
        C.c_void_p, _p_f64, _p_u8, _p_f64, _p_i32, _p_f32, _p_i32, _p_i32, _p_i32, _p_f32, _p_i32,
        C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_double,
        _p_i32, _p_i32, _p_i32, _p_i32]),
}

_lib = None


def load():
    """Loads libmmsim.so and declares every entry point.  Raises if it is absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} not found: build it with `python -m mms_amd.csrc.build` "
                "(hipcc, gfx950). mms_amd has no CPU fallback.")
        lib = C.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)      # AttributeError if the symbol is missing
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(rc):
    if rc != MMSIM_OK:
        raise MmsimError(rc, (load().mmsim_last_error() or b"").decode("utf-8", "replace"))


def ptr(arr, ctype):
    if arr is None:
        return None
    return arr.ctypes.data_as(C.POINTER(ctype))


def carray(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)
