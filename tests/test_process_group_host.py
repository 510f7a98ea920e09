"""CPU-side checks of the drop-in surface: `import fairring` registers the
backend, the options mirror fairring/bindings.cc:24-38, and contract violations
end the process like the reference's MY_CHECK (fairring/utils.h:29-33)."""
import datetime
import os
import subprocess
import sys

import pytest
import torch
import torch.distributed as dist

from conftest import ROOT

fairring = pytest.importorskip("fairring")
from fairring_amd import _fairring  # noqa: E402

MiB = 1024 * 1024


def make_pg(rank=0, size=1, **kw):
    o = _fairring.ProcessGroup.Options(
        max_memory_allocated_in_bytes=kw.pop("total", 50 * MiB),
        max_padding_allocated_in_bytes=kw.pop("padding", MiB),
        min_parallelism=kw.pop("parallelism", 16),
        is_high_priority_stream=True,
        timeout=datetime.timedelta(seconds=30), **kw)
    return _fairring.ProcessGroup(dist.HashStore(), rank, size, o)


def test_backend_is_registered():
    assert "fairring" in dist.Backend.backend_list
    assert dist.Backend.FAIRRING == "fairring"
    assert sys.modules["_fairring"] is _fairring


def test_process_group_surface():
    pg = make_pg(3, 8)
    assert isinstance(pg, torch._C._distributed_c10d.Backend)
    assert pg.name() == "fairring" and pg.rank() == 3 and pg.size() == 8
    with pytest.raises(TypeError):
        _fairring.ProcessGroup.Options(1, 2)  # min_parallelism is required
    o = _fairring.ProcessGroup.Options(50 * MiB, MiB, 16)  # positional, defaults for the rest
    assert o is not None
    with pytest.raises(RuntimeError):
        make_pg(8, 8)  # rank outside the group


def test_creator_reads_environment(monkeypatch, capsys):
    monkeypatch.delenv("FAIRRING_TOTAL_MEMORY", raising=False)
    pg = fairring.create_process_group_fairring(dist.HashStore(), 0, 1,
                                                datetime.timedelta(seconds=5))
    assert pg.name() == "fairring"
    assert "FAIRRING_TOTAL_MEMORY" in capsys.readouterr().err
    monkeypatch.setenv("FAIRRING_TOTAL_MEMORY", str(100 * MiB))
    monkeypatch.setenv("FAIRRING_SLICE_SIZE", str(25 * MiB))
    fairring.create_process_group_fairring(dist.HashStore(), 0, 1, datetime.timedelta(seconds=5))
    assert capsys.readouterr().err == ""


def _run(code):
    env = dict(os.environ, PYTHONPATH=ROOT)
    return subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True,
                          timeout=120)


PRELUDE = """
import datetime, torch, torch.distributed as dist
import fairring
from fairring_amd import _fairring
o = _fairring.ProcessGroup.Options(50 << 20, 1 << 20, 16)
pg = _fairring.ProcessGroup(dist.HashStore(), 0, 1, o)
"""


def test_cpu_tensor_terminates_like_my_check():
    r = _run(PRELUDE + "pg.allreduce([torch.zeros(4)])\nprint('survived')\n")
    assert r.returncode != 0 and "survived" not in r.stdout
    assert "Condition t.is_cuda() is false" in r.stderr


def test_sparse_tensor_terminates():
    r = _run(PRELUDE + "pg.allreduce([torch.zeros(8).to_sparse()])\nprint('survived')\n")
    assert r.returncode != 0 and "survived" not in r.stdout
    assert "t.layout() == at::kStrided" in r.stderr


def test_two_tensors_terminate():
    r = _run(PRELUDE + "pg.allreduce([torch.zeros(4), torch.zeros(4)])\nprint('survived')\n")
    assert r.returncode != 0 and "data.size() == 1" in r.stderr


def test_init_process_group_world_size_one():
    code = """
import torch, torch.distributed as dist
import fairring
dist.init_process_group("fairring", store=dist.HashStore(), rank=0, world_size=1)
assert dist.get_backend() == "fairring", dist.get_backend()
print("backend", dist.get_backend(), dist.get_world_size())
dist.destroy_process_group()
"""
    r = _run(code)
    assert r.returncode == 0, r.stderr
    assert "backend fairring 1" in r.stdout


def test_data_moving_collectives_for_a_group_of_one_on_cpu_tensors():
    # nothing moves in a group of one, so these need no GPU: enough to build DDP on the backend
    pg = make_pg(0, 1)
    x = torch.arange(100, dtype=torch.float32)
    w = pg.broadcast([x])
    assert w.wait() and w.is_completed() and w.is_success()
    out = torch.zeros(100)
    pg.allgather([[out]], [x]).wait()
    assert torch.equal(out, x)
    out2 = torch.zeros(4, 25)
    pg._allgather_base(out2, x).wait()
    assert torch.equal(out2.reshape(-1), x)
    assert pg.barrier().wait()
    pg2 = make_pg(1, 2)
    for call in (lambda: pg2.broadcast([x]), lambda: pg2.allgather([[out, out]], [x]),
                 lambda: pg2._allgather_base(torch.zeros(200), x), pg2.barrier):
        with pytest.raises(RuntimeError, match="needs a transport"):
            call()


def test_hook_entry_points_exist_and_refuse_other_backends():
    from fairring_amd import ddp_comm_hooks
    pg = make_pg(0, 1)
    assert hasattr(pg, "_allreduce_pre_divided") and hasattr(pg, "_allreduce_compressed")

    class Bucket:
        def buffer(self):
            return torch.zeros(4)

    for hook in (ddp_comm_hooks.allreduce_hook, ddp_comm_hooks.bf16_compress_hook,
                 ddp_comm_hooks.fp16_compress_hook):
        with pytest.raises(RuntimeError, match="'fairring' backend"):
            hook(object(), Bucket())


def test_simulated_peers_are_checked_when_they_are_set():
    # the peers' tensors are validated and flattened once, by the setter, not by every operation
    pg = make_pg(0, 3)
    with pytest.raises(RuntimeError, match="dense"):
        pg._set_simulated_peer_contributions([torch.zeros(8)[::2], torch.zeros(4)])
    with pytest.raises(RuntimeError, match="pinned"):
        pg._set_simulated_peer_contributions([torch.zeros(4), torch.zeros(4)])   # pageable memory
    pg._set_simulated_peer_contributions([])                                      # clears them
