"""TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Python face of the CPU oracle for Fairring's K-way gradient-slice reduction:
a ctypes binding of ``oracle.c`` plus an independent numpy restatement of the
same arithmetic. Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this package; the shipped
library (``fairring_amd``) never does.

Reference lines followed: fairring/device.cc:108-131 (doReduction),
fairring/device.cc:315-326 (slicing), fairring/utils.h:258-327 (layout).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

SCALE_NONE, SCALE_MUL, SCALE_DIV = 0, 1, 2
SCALE_PRE_MUL, SCALE_PRE_DIV = 3, 4  # every contribution scaled (and rounded) before the fold

_lib = None


def build(force=False):
    """Compile oracle.c with the Makefile beside it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, i32, f32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p
        for name in ("orc_sum_f32", "orc_sum_f32_chain", "orc_sum_bf16"):
            getattr(L, name).argtypes = [vp, vp, i32, i64, i32, f32]
            getattr(L, name).restype = None
        for name in ("orc_sum_f16", "orc_sum_f64"):
            getattr(L, name).argtypes = [vp, vp, i32, i64, i32, f32]
            getattr(L, name).restype = None
        for name in ("orc_max_f32", "orc_max_bf16", "orc_max_f16", "orc_max_f64",
                     "orc_sum_i32", "orc_max_i32", "orc_sum_i64", "orc_max_i64",
                     "orc_sum_u8", "orc_max_u8", "orc_sum_i8", "orc_max_i8"):
            getattr(L, name).argtypes = [vp, vp, i32, i64]
            getattr(L, name).restype = None
        L.orc_compressed_sum.argtypes = [vp, i32, vp, i32, i32, i64, i32, i32, f32]
        L.orc_compressed_sum.restype = None
        L.orc_ceil_of_ratio.argtypes = [i64, i64]
        L.orc_ceil_of_ratio.restype = i64
        L.orc_round_down.argtypes = [i64, i64]
        L.orc_round_down.restype = i64
        L.orc_round_up.argtypes = [i64, i64]
        L.orc_round_up.restype = i64
        L.orc_compute_layout.argtypes = [i64, i64, i64, i64, i64, vp]
        L.orc_compute_layout.restype = i32
        L.orc_readme_layout.argtypes = [i64, i64]
        L.orc_readme_layout.restype = i64
        L.orc_num_slices.argtypes = [i64, i64, i64]
        L.orc_num_slices.restype = i64
        L.orc_slice_bounds.argtypes = [i64, i64, i64, i64, vp]
        L.orc_slice_bounds.restype = None
        L.orc_set_threads.argtypes = [i32]
        L.orc_max_threads.restype = i32
        _lib = L
    return _lib


def _ptr_table(arrays):
    tab = (ctypes.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])
    return tab


def _prep(contribs, dtype):
    arrs = [np.ascontiguousarray(c, dtype=dtype).reshape(-1) for c in contribs]
    n = arrs[0].size
    assert all(a.size == n for a in arrs)
    return arrs, n


def sum_f32(contribs, scale_mode=SCALE_NONE, scale=1.0, chain=False, threads=1):
    """Sequential fp32 chain over a list of float32 arrays (C oracle)."""
    arrs, n = _prep(contribs, np.float32)
    out = np.empty(n, np.float32)
    L = lib()
    L.orc_set_threads(threads)
    fn = L.orc_sum_f32_chain if chain else L.orc_sum_f32
    fn(out.ctypes.data, _ptr_table(arrs), len(arrs), n, scale_mode, scale)
    return out


def sum_bf16(contribs, scale_mode=SCALE_NONE, scale=1.0, threads=1):
    """contribs: uint16 arrays holding bf16 bit patterns. Returns uint16."""
    arrs, n = _prep(contribs, np.uint16)
    out = np.empty(n, np.uint16)
    L = lib()
    L.orc_set_threads(threads)
    L.orc_sum_bf16(out.ctypes.data, _ptr_table(arrs), len(arrs), n, scale_mode, scale)
    return out


def max_f32(contribs):
    arrs, n = _prep(contribs, np.float32)
    out = np.empty(n, np.float32)
    lib().orc_max_f32(out.ctypes.data, _ptr_table(arrs), len(arrs), n)
    return out


def max_bf16(contribs):
    arrs, n = _prep(contribs, np.uint16)
    out = np.empty(n, np.uint16)
    lib().orc_max_bf16(out.ctypes.data, _ptr_table(arrs), len(arrs), n)
    return out


# name -> (numpy storage dtype, takes a post-scale)
TYPES = {"f32": (np.float32, True), "bf16": (np.uint16, True), "f16": (np.uint16, True),
         "f64": (np.float64, True), "i32": (np.int32, False), "i64": (np.int64, False),
         "u8": (np.uint8, False), "i8": (np.int8, False)}


def reduce(kind, contribs, op="sum", scale_mode=SCALE_NONE, scale=1.0):
    """Any element type by name ("f32", "bf16", "f16", "f64", "i32", "i64", "u8",
    "i8"); bf16 and f16 are passed as uint16 bit patterns."""
    npdt, scalable = TYPES[kind]
    arrs, n = _prep(contribs, npdt)
    out = np.empty(n, npdt)
    L = lib()
    L.orc_set_threads(1)
    fn = getattr(L, "orc_%s_%s" % (op, kind))
    if op == "sum" and scalable:
        fn(out.ctypes.data, _ptr_table(arrs), len(arrs), n, scale_mode, scale)
    else:
        assert scale_mode == SCALE_NONE
        fn(out.ctypes.data, _ptr_table(arrs), len(arrs), n)
    return out


def gathered_reduce(kind, contribs, gathered_index, segments, op="sum", scale_mode=SCALE_NONE,
                    scale=1.0):
    """The allreduce of a bucket whose own contribution still lies in separate
    gradient tensors: what the per-bucket allreduce of
    fairring/process_group.cc:131-155 returns after DDP has copied every gradient
    to its place in the bucket (torch:csrc/distributed/c10d/reducer.cpp,
    copy_grad_to_bucket: bucket_view.copy_(grad), views laid end to end in the
    flat bucket). `segments` are those tensors in bucket order; their
    concatenation takes the place of contribs[gathered_index] (ignored, may be
    None); the rest is `reduce`."""
    npdt, _ = TYPES[kind]
    own = (np.concatenate([np.ascontiguousarray(s, dtype=npdt).reshape(-1) for s in segments])
           if segments else np.empty(0, npdt))
    full = [own if k == gathered_index else c for k, c in enumerate(contribs)]
    return reduce(kind, full, op, scale_mode, scale)


def compressed_sum(contribs, raw_index, wire="bf16", scale_mode=SCALE_NONE, scale=1.0,
                   out_f32=True, threads=1):
    """torch's compress hook + allreduce + decompress for one rank's bucket.

    contribs[raw_index] is this rank's float32 buffer (raw_index -1: none), the
    others are uint16 arrays of wire-type bit patterns. Returns float32 (the
    decompressed bucket) or uint16 wire bits."""
    arrs = []
    for k, c in enumerate(contribs):
        dt = np.float32 if k == raw_index else np.uint16
        arrs.append(np.ascontiguousarray(c, dtype=dt).reshape(-1))
    n = arrs[0].size
    assert all(a.size == n for a in arrs)
    out = np.empty(n, np.float32 if out_f32 else np.uint16)
    L = lib()
    L.orc_set_threads(threads)
    L.orc_compressed_sum(out.ctypes.data, 1 if out_f32 else 0, _ptr_table(arrs), len(arrs),
                         raw_index, n, {"bf16": 0, "f16": 1}[wire], scale_mode, scale)
    return out


def compute_layout(max_mem, max_pad, min_par, num_machines, devs_per_machine):
    """Returns dict, or raises ValueError where the reference terminates."""
    out = (ctypes.c_int64 * 4)()
    rc = lib().orc_compute_layout(max_mem, max_pad, min_par, num_machines,
                                  devs_per_machine, out)
    if rc != 0:
        raise ValueError("computeLayout check %d failed" % rc)
    return dict(slot=out[0], slice=out[1], padding_slots=out[2], staging_slots=out[3])


def num_slices(numel, slice_bytes, elsize):
    return lib().orc_num_slices(numel, slice_bytes, elsize)


def slice_bounds(numel, slice_bytes, elsize, idx):
    out = (ctypes.c_int64 * 2)()
    lib().orc_slice_bounds(numel, slice_bytes, elsize, idx, out)
    return out[0], out[1]


# ---- independent numpy restatement ------------------------------------------

def np_bf16_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def np_f32_to_bf16_rne(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    bias = np.uint32(0x7FFF) + ((u >> 16) & np.uint32(1))
    r = ((u.astype(np.uint64) + bias) >> 16).astype(np.uint16)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    return np.where(nan, np.uint16(0x7FC0), r)


def _np_scale(acc, scale_mode, scale):
    if scale_mode == SCALE_MUL:
        return acc * np.float32(scale)
    if scale_mode == SCALE_DIV:
        return acc / np.float32(scale)
    return acc


def np_sum_f32(contribs, scale_mode=SCALE_NONE, scale=1.0):
    with np.errstate(all="ignore"):
        acc = np.array(contribs[0], np.float32, copy=True).reshape(-1)
        for c in contribs[1:]:
            acc = acc + np.asarray(c, np.float32).reshape(-1)
        return _np_scale(acc, scale_mode, scale).astype(np.float32)


def np_sum_bf16(contribs, scale_mode=SCALE_NONE, scale=1.0):
    with np.errstate(all="ignore"):
        acc = np_bf16_to_f32(np.asarray(contribs[0], np.uint16).reshape(-1)).copy()
        for c in contribs[1:]:
            acc = acc + np_bf16_to_f32(np.asarray(c, np.uint16).reshape(-1))
        return np_f32_to_bf16_rne(_np_scale(acc, scale_mode, scale))
