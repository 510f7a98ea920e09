"""MI355X-native K-way gradient-slice reduction behind Fairring's allreduce surface.

The compute path is libfairring_hip.so (hand-written gfx950 kernels + a HIP
stream/event slice pipeline) reached through the C ABI of
include/fairring_hip.h; importing this package does not load it, using it does,
and a missing library is an error, never a fallback.
"""
from ._capi import (BF16, F32, MAX, SCALE_DIV, SCALE_MUL, SCALE_NONE, SUM,  # noqa: F401
                    FairringError)
from .device import (DeviceFairring, Work, compute_layout, options_from_env,  # noqa: F401
                     reduce_slice)

__all__ = ["DeviceFairring", "Work", "FairringError", "compute_layout", "options_from_env",
           "reduce_slice", "F32", "BF16", "SUM", "MAX", "SCALE_NONE", "SCALE_MUL", "SCALE_DIV"]
