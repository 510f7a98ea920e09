import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# A wait that sees no progress for a minute ends in an error that says where the
# pipeline stands, instead of a silent stall (read when the libraries load).
os.environ.setdefault("FAIRRING_WAIT_TIMEOUT_S", "60")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden():
    path = os.path.join(ROOT, "tests", "golden", "ksum_golden.npz")
    with np.load(path, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def bits32(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def assert_bits_equal(a, b, what="", half=False):
    """Bit-exact comparison; any NaN payload counts as equal to any NaN. uint16
    arrays hold bf16 bit patterns, or fp16 ones with half=True."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    assert a.shape == b.shape, (what, a.shape, b.shape)
    assert a.dtype == b.dtype, (what, a.dtype, b.dtype)
    if a.dtype == np.float32:
        ua, ub = a.view(np.uint32), b.view(np.uint32)
        both_nan = np.isnan(a) & np.isnan(b)
    elif a.dtype == np.float64:
        ua, ub = a.view(np.uint64), b.view(np.uint64)
        both_nan = np.isnan(a) & np.isnan(b)
    elif a.dtype == np.uint16:
        ua, ub = a, b
        top = 0x7C00 if half else 0x7F80
        both_nan = ((a & 0x7FFF) > top) & ((b & 0x7FFF) > top)
    else:
        ua, ub = a, b
        both_nan = np.zeros(a.shape, bool)
    bad = (ua != ub) & ~both_nan
    if bad.any():
        i = int(np.flatnonzero(bad)[0])
        raise AssertionError("%s: %d mismatches, first at %d: %r vs %r" % (
            what, int(bad.sum()), i, ua.reshape(-1)[i], ub.reshape(-1)[i]))
