"""MI355X-native K-way gradient-slice reduction behind Fairring's allreduce surface.

The compute path is libfairring_hip.so (hand-written gfx950 kernels + a HIP
stream/event slice pipeline) reached through the C ABI of
include/fairring_hip.h; importing this package does not load it, using it does,
and a missing library is an error, never a fallback.
"""
from ._capi import (BF16, F16, F32, F64, I8, I32, I64, MAX, SCALE_DIV,  # noqa: F401
                    SCALE_MUL, SCALE_NONE, SCALE_PRE_DIV, SCALE_PRE_MUL, SUM, U8, FairringError)
from .device import (DeviceFairring, Work, compute_layout, options_from_env, plan_launches,  # noqa: F401
                     reduce_pieces, reduce_slice, reduce_slice_compressed, reduce_slice_static,
                     set_wait_timeout)

__all__ = ["DeviceFairring", "Work", "FairringError", "compute_layout", "options_from_env", "plan_launches",
           "reduce_pieces", "reduce_slice", "reduce_slice_compressed", "reduce_slice_static", "set_wait_timeout", "F32", "BF16", "F16", "F64", "I32", "I64",
           "U8", "I8", "SUM", "MAX", "SCALE_NONE", "SCALE_MUL", "SCALE_DIV", "SCALE_PRE_MUL",
           "SCALE_PRE_DIV"]
