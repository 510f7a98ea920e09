"""CPU-side checks: the C-ABI library loads and exports every symbol that
include/fairring_hip.h declares, and its pure host logic (layout, slicing,
environment parsing, argument validation) agrees with the oracle. No GPU call.
"""
import ctypes
import io
import os
import re

import pytest

import oracle
from conftest import ROOT

fa = pytest.importorskip("fairring_amd")
from fairring_amd import _capi  # noqa: E402

MiB = 1024 * 1024


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "fairring_hip.h")).read()
    return sorted(set(re.findall(r"FRG_API[^;(]*?\b(frg_[a-z_0-9]+)\s*\(", text)))


def test_header_symbols_are_exported():
    L = _capi.lib()
    names = declared_symbols()
    assert len(names) >= 19
    for n in names:
        assert hasattr(L, n), "library does not export " + n
    assert sorted(_capi.EXPORTS) == names


def test_version_and_error_string():
    L = _capi.lib()
    assert re.match(rb"^\d+\.\d+$", L.frg_version())
    lay = _capi.Layout()
    rc = L.frg_compute_layout(50 * MiB, 64, 16, 1, 1, ctypes.byref(lay))
    assert rc == _capi.ERR_LAYOUT
    assert b"padding" in L.frg_last_error()


@pytest.mark.parametrize("args", [
    (50 * MiB, MiB, 16, 1, 1), (50 * MiB, MiB, 16, 8, 1), (50 * MiB, MiB, 2, 1, 1),
    (50 * MiB, MiB, 16, 4, 8), (123456789, 4 * MiB, 7, 3, 1), (MiB, MiB, 1, 64, 1)])
def test_layout_matches_oracle(args):
    assert fa.compute_layout(*args) == oracle.compute_layout(*args)


@pytest.mark.parametrize("args", [(50 * MiB, 64, 16, 1, 1), (100, MiB, 16, 1, 1)])
def test_layout_failures_match_oracle(args):
    with pytest.raises(ValueError):
        oracle.compute_layout(*args)
    with pytest.raises(fa.FairringError) as e:
        fa.compute_layout(*args)
    assert e.value.code == _capi.ERR_LAYOUT


def test_slicing_matches_oracle_and_known_answers():
    L = _capi.lib()
    S = 25 * MiB
    assert L.frg_num_slices(1_370_000_000, S, 4) == 210
    assert L.frg_num_slices(1_300_000_000, S, 2) == 100
    assert L.frg_num_slices(0, S, 4) == 0
    off, ln = ctypes.c_int64(), ctypes.c_int64()
    for numel, sb, es in [(1_370_000_000, S, 4), (1_300_000_000, S, 2), (1001, 96, 4), (5, 8, 2)]:
        n = L.frg_num_slices(numel, sb, es)
        assert n == oracle.num_slices(numel, sb, es)
        for i in {0, n // 2, n - 1}:
            assert L.frg_slice_bounds(numel, sb, es, i, ctypes.byref(off), ctypes.byref(ln)) == 0
            assert (off.value, ln.value) == oracle.slice_bounds(numel, sb, es, i)
    assert L.frg_slice_bounds(10, 8, 4, 5, ctypes.byref(off), ctypes.byref(ln)) == _capi.ERR_INVALID


def test_options_from_env_defaults_and_notice():
    err = io.StringIO()
    o = fa.options_from_env({}, err)
    assert o == dict(max_memory_allocated_in_bytes=50 * MiB,
                     max_padding_allocated_in_bytes=MiB, min_parallelism=16)
    assert "FAIRRING_TOTAL_MEMORY" in err.getvalue() and "50 MiB" in err.getvalue()
    err = io.StringIO()
    o = fa.options_from_env({"FAIRRING_TOTAL_MEMORY": "1000000", "FAIRRING_PARALLELISM": "2",
                             "FAIRRING_PADDING_MEMORY": "4096", "FAIRRING_SLICE_SIZE": "4000"}, err)
    assert o == dict(max_memory_allocated_in_bytes=1000000, max_padding_allocated_in_bytes=4096,
                     min_parallelism=2, slice_size_in_bytes=4000)
    assert err.getvalue() == ""


def test_reduce_slice_rejects_bad_arguments_before_touching_the_gpu():
    L = _capi.lib()
    tab = _capi.ptr_table([16, 32])
    assert L.frg_reduce_slice(64, tab, 0, 4, 0, 0, 0, 1.0, 0, None) == _capi.ERR_INVALID
    assert L.frg_reduce_slice(64, tab, 2, 4, 8, 0, 0, 1.0, 0, None) == _capi.ERR_UNSUPPORTED  # dtype code
    assert L.frg_reduce_slice(64, tab, 2, 4, 4, 0, 1, 0.5, 0, None) == _capi.ERR_INVALID  # int32 with a scale
    assert L.frg_reduce_slice(64, tab, 2, 4, 0, 3, 0, 1.0, 0, None) == _capi.ERR_UNSUPPORTED
    assert L.frg_reduce_slice(64, tab, 2, -1, 0, 0, 0, 1.0, 0, None) == _capi.ERR_INVALID
    assert L.frg_reduce_slice(64, tab, 2, 4, 0, 1, 1, 0.5, 0, None) == _capi.ERR_INVALID
    assert L.frg_reduce_slice(64, tab, 2, 0, 0, 0, 0, 1.0, 0, None) == _capi.OK  # empty: no-op
    assert L.frg_reduce_slice(None, tab, 2, 4, 0, 0, 0, 1.0, 0, None) == _capi.ERR_INVALID
    assert L.frg_reduce_slice(66, tab, 2, 4, 0, 0, 0, 1.0, 0, None) == _capi.ERR_INVALID  # misaligned
    assert L.frg_reduce_slice(24, tab, 2, 4, 0, 0, 0, 1.0, 0, None) == _capi.ERR_INVALID  # overlap


def test_create_without_gpu_fails_cleanly():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(fa.FairringError) as e:
        fa.DeviceFairring(0)
    assert e.value.code == _capi.ERR_HIP


def test_dense_check():
    import torch
    from fairring_amd.device import is_non_overlapping_and_dense as dense
    assert dense(torch.zeros(3, 4)) and dense(torch.zeros(3, 4).t())
    assert dense(torch.zeros(2, 3, 4).permute(2, 0, 1))
    assert not dense(torch.zeros(3, 4)[:, :2]) and not dense(torch.zeros(8)[::2])
    assert dense(torch.zeros(0))


def test_header_is_plain_c(tmp_path):
    # the boundary is a C ABI: the header must compile as strict C99 on its own
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("gcc not available")
    src = tmp_path / "use_header.c"
    src.write_text('#include "fairring_hip.h"\n'
                   "int probe(void) { frg_options o = {0}; frg_progress p = {0}; frg_progress2 q = {0};\n"
                   "  return (int)(o.num_machines + p.launches + q.segmented_launches + sizeof(q))\n"
                   "         + FRG_SCALE_PRE_DIV + FRG_I8; }\n")
    r = subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only",
                        "-I", os.path.join(ROOT, "include"), str(src)],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr


def test_c_client_builds_and_fails_cleanly_without_a_gpu(tmp_path):
    import shutil
    import subprocess
    import torch
    if shutil.which("gcc") is None:
        pytest.skip("gcc not available")
    from fairring_amd import build as hip_build
    exe = hip_build.build_c_client(str(tmp_path / "abi_client"))
    # rpath of the copy does not reach the library: point the loader at it
    env = dict(os.environ, LD_LIBRARY_PATH=os.path.join(ROOT, "fairring_amd") + ":" +
               os.environ.get("LD_LIBRARY_PATH", ""))
    r = subprocess.run([exe, "2", "100"], capture_output=True, text=True, timeout=120, env=env)
    if torch.cuda.is_available():
        assert r.returncode == 0 and "abi client ok" in r.stdout, r.stderr
    else:
        assert r.returncode == 2 and "abi 0.3" in r.stdout     # the HIP runtime finds no device


def test_a_missing_library_is_a_loud_error_not_a_fallback(tmp_path):
    # the product path has no CPU implementation to fall back on: without the built library
    # the first use raises and names the build command
    import subprocess
    import sys
    code = ("import fairring_amd as fa\n"
            "try:\n"
            "    fa.compute_layout(50 << 20, 1 << 20, 16, 1, 1)\n"
            "except ImportError as e:\n"
            "    print('raised:', e)\n")
    env = dict(os.environ, PYTHONPATH=ROOT, FAIRRING_HIP_LIBRARY=str(tmp_path / "absent.so"))
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    assert "raised:" in r.stdout and "no fallback" in r.stdout and "fairring_amd.build" in r.stdout
    # and the package never imports the oracle
    src = "".join(open(os.path.join(ROOT, "fairring_amd", f)).read()
                  for f in os.listdir(os.path.join(ROOT, "fairring_amd")) if f.endswith(".py"))
    assert "import oracle" not in src and "from oracle" not in src
