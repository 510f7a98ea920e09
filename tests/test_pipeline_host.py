"""Host logic of the slice pipeline on a CPU stand-in for the HIP runtime
(tests/host/fake_hip): slicing and launch splitting, stream rotation, the
initial-event rule, staging-slot reuse, carry chains, completion callbacks,
injected HIP failures, profile marks, destruction with work pending and
concurrent submitters; each on two models of how a stream wait binds to its event. Built three ways: plain, ThreadSanitizer, and
AddressSanitizer + UBSan. No GPU, no reference code; the reduction itself is
a plain fp32 fold inside the test build, so only the choreography is under
test here (kernel parity is the GPU suite's job).
"""
import os
import shutil
import subprocess

import pytest

from conftest import ROOT

HOST = os.path.join(ROOT, "tests", "host")
SOURCES = [
    os.path.join(HOST, "pipeline_host_test.cc"),
    os.path.join(HOST, "ksum_host.cc"),
    os.path.join(HOST, "fake_hip", "fake_hip.cc"),
    os.path.join(ROOT, "fairring_amd", "csrc", "pipeline.cc"),
    os.path.join(ROOT, "fairring_amd", "csrc", "schedule_resident.cc"),
    os.path.join(ROOT, "fairring_amd", "csrc", "schedule_gathered.cc"),
    os.path.join(ROOT, "fairring_amd", "csrc", "schedule_host_staged.cc"),
    os.path.join(ROOT, "fairring_amd", "csrc", "capi.cc"),
]

VARIANTS = {
    "plain": [],
    "tsan": ["-fsanitize=thread"],
    "asan_ubsan": ["-fsanitize=address,undefined", "-fno-sanitize-recover=all"],
}


_built = {}


def _build(variant, tmp_path_factory):
    """The scenarios' executable for one sanitizer variant, built once per session."""
    if variant not in _built:
        exe = str(tmp_path_factory.mktemp("host") / ("pipeline_host_" + variant))
        cmd = ["g++", "-std=c++17", "-O1", "-g", "-pthread", "-Wall", "-I",
               os.path.join(HOST, "fake_hip")] + VARIANTS[variant] + ["-o", exe] + SOURCES
        build = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        assert build.returncode == 0, build.stderr[-4000:]
        _built[variant] = exe
    return _built[variant]


# Every scenario on two models of the runtime: one whose stream waits bind to the record their
# event held when the wait was enqueued (what HIP does; measured on the MI355X), and one where
# they bind to the record the event holds when the wait is executed. The pipeline records every
# event once, so it must come out the same on both.
@pytest.mark.timeout(400)
@pytest.mark.parametrize("waits", ["bound-at-enqueue", "latest-record-waits"])
@pytest.mark.parametrize("variant", list(VARIANTS))
def test_pipeline_host_scenarios(variant, waits, tmp_path_factory):
    if shutil.which("g++") is None:
        pytest.skip("g++ not available")
    exe = _build(variant, tmp_path_factory)
    env = dict(os.environ,
               TSAN_OPTIONS="halt_on_error=1 second_deadlock_stack=1",
               # the pipeline leaks its streams on purpose (consumers may still hold events
               # ordered after them), so leak checking is off
               ASAN_OPTIONS="detect_leaks=0 abort_on_error=1",
               UBSAN_OPTIONS="print_stacktrace=1")
    # ThreadSanitizer slows the scenarios tenfold; it runs them in the topology of a GPU
    # process (4 shared hardware queues) only: what it looks for does not depend on that
    if variant == "tsan":
        env["HOST_TEST_TOPOLOGY"] = "4"
    mode = [waits] if waits == "latest-record-waits" else []
    run = subprocess.run([exe] + mode, capture_output=True, text=True, timeout=380, env=env)
    assert run.returncode == 0, (run.stdout[-2000:], run.stderr[-4000:])
    assert "ALL HOST SCENARIOS PASSED" in run.stdout
    assert "WARNING: ThreadSanitizer" not in run.stderr
