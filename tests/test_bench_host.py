"""bench.py's host-side logic, no GPU: the refusal of more than one GPU, the
launch-size rule it reports (which must be the pipeline's own), the bucket
schedule of the DDP workload and the interval arithmetic behind the roofline."""
import os
import subprocess
import sys
import types

import pytest

from conftest import ROOT

sys.path.insert(0, ROOT)
import bench  # noqa: E402

MiB = 1024 * 1024


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_defaults_are_the_headline_configuration():
    old = sys.argv
    sys.argv = ["bench.py"]
    try:
        a = bench.parse_args()
    finally:
        sys.argv = old
    assert (a.gpus, a.workload, a.slice_bytes, a.total_memory) == (1, "c2", 25 * MiB, 50 * MiB)
    assert a.steps >= 1 and a.warmup >= 1
    # the driver's record carries every other workload of the benchmark definition too
    assert sorted(a.extras.split(",")) == sorted(["c5", "c5pg", "c5sep", "gather", "c4", "hook", "c3"])


@pytest.mark.parametrize("op_elems,slice_elems,elsize,lb,want", [
    (1_370_000_000, 6_553_600, 4, 0, 2_097_152),   # a whole fp32 gradient: 8 MiB launches, whatever the slice size
    (1_300_000_000, 13_107_200, 2, 0, 4_194_304),  # bf16: the same 8 MiB
    (1_370_000_000, 819_196, 4, 0, 2_097_152),     # default layout (3,276,784 B slices): the same
    (1_370_000_000, 6_553_600, 4, -1, 6_553_600),  # one launch per slice
    (6_553_600, 6_553_600, 4, 0, 3_276_800),       # one 25 MiB bucket on its own: two launches
    (262_144, 6_553_600, 4, 0, 262_144),           # the 1 MiB bucket: one launch
    (4_000_000, 6_553_600, 4, 0, 4_000_000),       # up to 1.5 x the launch size: still one launch
    (1_370_000_000, 6_553_600, 4, 6 * MiB, 1_572_864),
])
def test_launch_elems_follows_the_pipeline_rule(op_elems, slice_elems, elsize, lb, want):
    args = types.SimpleNamespace(launch_bytes=lb)
    assert bench.launch_elems(args, op_elems, slice_elems, elsize) == want


def test_ddp_bucket_schedule():
    spans = bench.ddp_buckets(1_370_000_000, 25 * MiB // 4, MiB // 4)
    assert len(spans) == 211
    assert spans[0] == (1_370_000_000 - 262_144, 1_370_000_000)      # the small first bucket
    assert spans[-1][0] == 0
    assert all(a[0] == b[1] for a, b in zip(spans, spans[1:]))        # released back to front
    assert sum(hi - lo for lo, hi in spans) == 1_370_000_000
    assert max(hi - lo for lo, hi in spans) == 25 * MiB // 4


def test_union_length_and_roofline_arithmetic():
    assert bench.union_length([]) == 0.0
    assert bench.union_length([(0, 1), (0.5, 2), (3, 4)]) == pytest.approx(3.0)
    assert bench.union_length([(3, 4), (0, 10)]) == pytest.approx(10.0)
    # two streams, each busy for the same 10 ms with 100 launches of 1e6 elements
    recs = [(0.0, 10.0, 100_000_000, 8, 0, 100), (0.0, 10.0, 100_000_000, 8, 1, 100)]
    roof = bench.roofline_from_records(recs, 36, 1_000_000, "how")
    assert roof["achieved"] == pytest.approx(2e8 * 36 / 10e-3 / 1e9, rel=1e-3)
    assert roof["concurrency"] == pytest.approx(2.0)
    assert roof["avg_launch_us"] == pytest.approx(100.0)
    assert roof["frac"] == pytest.approx(roof["achieved"] / 8000.0, rel=1e-3)
    assert roof["bound"] == "hbm" and roof["unit"] == "GB/s" and roof["peak"] == 8000.0
