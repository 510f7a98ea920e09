"""ctypes binding of the C ABI in include/fairring_hip.h.

Loading fails loudly when libfairring_hip.so has not been built: there is no
CPU or eager fallback behind this module.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libfairring_hip.so")

OK, ERR_INVALID, ERR_HIP, ERR_LAYOUT, ERR_UNSUPPORTED, ERR_NOT_READY = range(6)
F32, BF16, F16, F64, I32, I64, U8, I8 = range(8)
SUM, MAX = 0, 1
SCALE_NONE, SCALE_MUL, SCALE_DIV = 0, 1, 2
SCALE_PRE_MUL, SCALE_PRE_DIV = 3, 4

# every symbol include/fairring_hip.h declares
EXPORTS = (
    "frg_compute_layout", "frg_num_slices", "frg_slice_bounds", "frg_plan_launches", "frg_reduce_slice", "frg_reduce_slice_static",
    "frg_reduce_slice_compressed", "frg_allreduce_compressed",
    "frg_create", "frg_destroy", "frg_get_layout", "frg_get_streams", "frg_get_copy_streams", "frg_allreduce", "frg_allreduce_host",
    "frg_work_wait", "frg_set_wait_timeout", "frg_get_progress", "frg_get_progress2", "frg_allreduce_gathered", "frg_allreduce_compressed_gathered", "frg_reduce_pieces", "frg_work_is_completed", "frg_work_block_stream", "frg_work_release",
    "frg_synchronize", "frg_profile_mark", "frg_set_profiling", "frg_kernel_times", "frg_launch_records",
    "frg_set_tuning", "frg_set_tile_runs", "frg_set_mixed_loads",
    "frg_last_error", "frg_version",
)


class FairringError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("fairring error %d: %s" % (code, message))
        self.code = code


class Layout(ctypes.Structure):
    _fields_ = [("slot_size_in_bytes", ctypes.c_int64),
                ("slice_size_in_bytes", ctypes.c_int64),
                ("num_padding_slots", ctypes.c_int64),
                ("num_staging_slots", ctypes.c_int64)]


class Options(ctypes.Structure):
    _fields_ = [("max_memory_allocated_in_bytes", ctypes.c_int64),
                ("max_padding_allocated_in_bytes", ctypes.c_int64),
                ("min_parallelism", ctypes.c_int64),
                ("slice_size_in_bytes", ctypes.c_int64),
                ("num_machines", ctypes.c_int64),
                ("num_reduce_streams", ctypes.c_int32),
                ("num_copy_streams", ctypes.c_int32),
                ("max_launch_bytes", ctypes.c_int64)]


class Segment(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("numel", ctypes.c_int64)]


class Piece(ctypes.Structure):
    _fields_ = [("out", ctypes.c_void_p), ("contribs", ctypes.POINTER(ctypes.c_void_p)),
                ("numel", ctypes.c_int64)]


class LaunchRecord(ctypes.Structure):
    _fields_ = [("begin_ms", ctypes.c_float), ("end_ms", ctypes.c_float),
                ("numel", ctypes.c_int64), ("num_contributions", ctypes.c_int32),
                ("stream_index", ctypes.c_int32), ("launches", ctypes.c_int32),
                ("reserved", ctypes.c_int32)]


DONE_FN = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p)

_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    path = os.environ.get("FAIRRING_HIP_LIBRARY", LIB_PATH)
    if not os.path.exists(path):
        raise ImportError(
            "%s is missing: build it with `python -m fairring_amd.build` "
            "(there is no fallback implementation)" % path)
    # PyTorch ships its own copy of the HIP runtime. Load it first so that this
    # library binds to the runtime that owns torch's tensors and streams; two
    # runtimes in one process do not see each other's devices.
    import torch  # noqa: F401
    L = ctypes.CDLL(path)
    i64, i32, f32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p
    pvp = ctypes.POINTER(ctypes.c_void_p)
    L.frg_compute_layout.argtypes = [i64, i64, i64, i64, i64, ctypes.POINTER(Layout)]
    L.frg_num_slices.argtypes = [i64, i64, i64]
    L.frg_num_slices.restype = i64
    L.frg_slice_bounds.argtypes = [i64, i64, i64, i64, ctypes.POINTER(i64), ctypes.POINTER(i64)]
    L.frg_plan_launches.argtypes = [i32, i64, i64, ctypes.c_uint64, ctypes.c_uint64, i32, i32,
                                    ctypes.POINTER(i64),
                                    ctypes.POINTER(ctypes.c_int32), i32, ctypes.POINTER(i32)]
    L.frg_reduce_slice.argtypes = [vp, pvp, i32, i64, i32, i32, i32, f32, i32, vp]
    L.frg_reduce_slice_static.argtypes = [vp, pvp, i32, i64, i32, i32, i32, f32, vp]
    L.frg_create.argtypes = [i32, ctypes.POINTER(Options), pvp]
    L.frg_destroy.argtypes = [vp]
    L.frg_get_layout.argtypes = [vp, ctypes.POINTER(Layout)]
    L.frg_get_streams.argtypes = [vp, pvp, i32, ctypes.POINTER(i32)]
    L.frg_get_copy_streams.argtypes = [vp, pvp, i32, ctypes.POINTER(i32)]
    L.frg_allreduce.argtypes = [vp, vp, pvp, i32, i64, i32, i32, i32, f32, vp, DONE_FN, vp, pvp]
    L.frg_reduce_slice_compressed.argtypes = [vp, i32, pvp, i32, i32, i64, i32, i32, f32, vp]
    L.frg_allreduce_compressed.argtypes = [vp, vp, i32, pvp, i32, i32, i64, i32, i32, f32, vp,
                                           DONE_FN, vp, pvp]
    L.frg_allreduce_gathered.argtypes = [vp, vp, pvp, i32, i32, ctypes.POINTER(Segment), i32, i64,
                                         i32, i32, i32, f32, vp, DONE_FN, vp, pvp]
    L.frg_allreduce_compressed_gathered.argtypes = [vp, vp, i32, pvp, i32, i32,
                                                    ctypes.POINTER(Segment), i32, i64, i32, i32, f32,
                                                    vp, DONE_FN, vp, pvp]
    L.frg_reduce_pieces.argtypes = [ctypes.POINTER(Piece), i32, i32, i32, i32, i32, f32, vp]
    L.frg_allreduce_host.argtypes = [vp, vp, pvp, i32, i64, i32, i32, i32, f32, i32, vp,
                                     DONE_FN, vp, pvp]
    for fn in (L.frg_work_wait, L.frg_work_is_completed, L.frg_work_release, L.frg_synchronize,
               L.frg_profile_mark):
        fn.argtypes = [vp]
    L.frg_work_block_stream.argtypes = [vp, vp]
    L.frg_set_wait_timeout.argtypes = [ctypes.c_double]
    L.frg_get_progress.argtypes = [vp, ctypes.POINTER(ctypes.c_int64 * 4)]
    L.frg_get_progress2.argtypes = [vp, ctypes.POINTER(ctypes.c_int64 * 7), ctypes.c_uint64]
    L.frg_set_profiling.argtypes = [vp, i32]
    L.frg_kernel_times.argtypes = [vp, ctypes.POINTER(ctypes.c_float), i32, ctypes.POINTER(i32)]
    L.frg_launch_records.argtypes = [vp, ctypes.POINTER(LaunchRecord), i32, ctypes.POINTER(i32)]
    L.frg_set_tuning.argtypes = [i32]
    L.frg_set_tile_runs.argtypes = [i32]
    L.frg_set_mixed_loads.argtypes = [i32]
    L.frg_last_error.restype = ctypes.c_char_p
    L.frg_version.restype = ctypes.c_char_p
    _lib = L
    return L


def check(rc):
    if rc != OK:
        raise FairringError(rc, lib().frg_last_error().decode("utf-8", "replace"))


def ptr_table(ptrs):
    return (ctypes.c_void_p * len(ptrs))(*ptrs)
