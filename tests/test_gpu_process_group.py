"""GPU tests of the drop-in surface: `_fairring.ProcessGroup.allreduce` with
simulated peer contributions, against the CPU oracle (bit-exact)."""
import datetime
import os
import subprocess
import sys

import numpy as np
import pytest
import torch
import torch.distributed as dist

import oracle
from conftest import ROOT, assert_bits_equal

pytestmark = pytest.mark.gpu

fairring = pytest.importorskip("fairring")
from fairring_amd import _fairring  # noqa: E402

DEV = "cuda:0"
MiB = 1024 * 1024


def make_pg(rank, size, total=50 * MiB, parallelism=16, slice_bytes=0):
    o = _fairring.ProcessGroup.Options(
        max_memory_allocated_in_bytes=total, max_padding_allocated_in_bytes=MiB,
        min_parallelism=parallelism, is_high_priority_stream=True,
        timeout=datetime.timedelta(seconds=60), slice_size_in_bytes=slice_bytes)
    return _fairring.ProcessGroup(dist.HashStore(), rank, size, o)


def ordered(own, peers, rank):
    return peers[:rank] + [own] + peers[rank:]


@pytest.mark.parametrize("rank,size", [(0, 2), (3, 8), (7, 8), (5, 17), (0, 64)])
def test_allreduce_sum_matches_oracle(rank, size):
    print("[case] pg sum", rank, size, flush=True)
    n = 300_007
    rng = np.random.default_rng(rank * 100 + size)
    x = (rng.standard_normal((size, n)) * 0.01).astype(np.float32)
    pg = make_pg(rank, size, slice_bytes=256 * 1024, total=MiB)
    own = torch.from_numpy(x[rank].copy()).to(DEV)
    peers = [torch.from_numpy(x[r].copy()).to(DEV) for r in range(size) if r != rank]
    pg._set_simulated_peer_contributions(peers)
    work = pg.allreduce([own])
    assert work.wait() is True
    assert work.is_completed() and work.is_success()
    torch.cuda.synchronize()
    assert_bits_equal(own.cpu().numpy(), oracle.sum_f32(list(x)))
    res = work.result()
    assert len(res) == 1 and res[0].data_ptr() == own.data_ptr()  # in place, borrowed
    assert pg._layout()[1] == 256 * 1024


def test_allreduce_fused_divide_and_future():
    print("[case] pg fused divide", flush=True)
    size, rank, n = 8, 2, 1_000_003
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((size, n)) * 0.01).astype(np.float32)
    pg = make_pg(rank, size)   # default layout: 16 slots of 3,276,784 B for M = 8 -> 3,276,672
    pg._set_fused_divide(True)
    own = torch.from_numpy(x[rank].copy()).to(DEV)
    pg._set_simulated_peer_contributions(
        [torch.from_numpy(x[r].copy()).to(DEV) for r in range(size) if r != rank])
    fut = pg.allreduce([own]).get_future()
    doubled = fut.then(lambda f: f.value()[0] * 2)   # ordered on the GPU after the reduction
    got2 = doubled.wait()
    torch.cuda.synchronize()
    want = oracle.sum_f32(list(x), oracle.SCALE_MUL, 0.125)
    assert_bits_equal(own.cpu().numpy(), want)
    assert_bits_equal(got2.cpu().numpy(), want * np.float32(2))
    assert pg._layout() == [3276672, 3276672, 16, 16]


def test_allreduce_non_power_of_two_divide():
    print("[case] pg divide by 3", flush=True)
    size, rank, n = 3, 1, 50_001
    rng = np.random.default_rng(6)
    x = rng.standard_normal((size, n)).astype(np.float32)
    pg = make_pg(rank, size)
    pg._set_fused_divide(True)
    own = torch.from_numpy(x[rank].copy()).to(DEV)
    pg._set_simulated_peer_contributions(
        [torch.from_numpy(x[r].copy()).to(DEV) for r in range(size) if r != rank])
    pg.allreduce([own]).wait()
    torch.cuda.synchronize()
    assert_bits_equal(own.cpu().numpy(), oracle.sum_f32(list(x), oracle.SCALE_DIV, 3.0))


def test_allreduce_bf16_and_max_and_permuted_dense():
    print("[case] pg bf16/max/permuted", flush=True)
    size, rank = 4, 0
    rng = np.random.default_rng(7)
    x = (rng.standard_normal((size, 64, 1000)) * 0.01).astype(np.float32)
    bits = oracle.np_f32_to_bf16_rne(x)
    pg = make_pg(rank, size)

    def dev_bf16(b):
        return torch.from_numpy(b.view(np.int16).copy()).to(DEV).view(torch.bfloat16)

    # a transposed (dense, non-contiguous) tensor is reduced over its storage order
    own = dev_bf16(bits[0]).t()
    peers = [dev_bf16(bits[r]).t() for r in range(1, size)]
    pg._set_simulated_peer_contributions(peers)
    pg.allreduce([own]).wait()
    torch.cuda.synchronize()
    got = own.t().contiguous().view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1)
    assert_bits_equal(got, oracle.sum_bf16([b.reshape(-1) for b in bits]))

    opts = dist.AllreduceOptions()
    opts.reduceOp = dist.ReduceOp.MAX
    own = torch.from_numpy(x[0].copy()).to(DEV)
    pg._set_simulated_peer_contributions([torch.from_numpy(x[r].copy()).to(DEV)
                                          for r in range(1, size)])
    pg.allreduce([own], opts).wait()
    torch.cuda.synchronize()
    assert_bits_equal(own.cpu().numpy().reshape(-1), oracle.max_f32([a.reshape(-1) for a in x]))


def test_allreduce_server_side_from_pinned_host():
    print("[case] pg pinned peers", flush=True)
    size, n = 16, 400_003
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((size, n)) * 0.01).astype(np.float32)
    pg = make_pg(0, size, total=2 * MiB, slice_bytes=MiB)   # 2 slots of 1 MiB
    pg._set_fused_divide(True)
    own = torch.from_numpy(x[0].copy()).to(DEV)
    pg._set_simulated_peer_contributions(
        [torch.from_numpy(x[r].copy()).pin_memory() for r in range(1, size)])
    pg.allreduce([own]).wait()
    torch.cuda.synchronize()
    assert_bits_equal(own.cpu().numpy(), oracle.sum_f32(list(x), oracle.SCALE_MUL, 1.0 / 16))


def test_missing_peers_is_a_loud_error():
    print("[case] pg missing peers", flush=True)
    pg = make_pg(0, 2)
    with pytest.raises(RuntimeError, match="simulated peer"):
        pg.allreduce([torch.zeros(10, device=DEV)])


def test_world_size_one_through_torch_distributed():
    print("[case] init_process_group", flush=True)
    code = """
import torch, torch.distributed as dist
import fairring
dist.init_process_group("fairring", store=dist.HashStore(), rank=0, world_size=1)
t = torch.arange(1000, dtype=torch.float32, device="cuda:0")
w = dist.all_reduce(t, async_op=True)
w.wait()
torch.cuda.synchronize()
assert bool((t == torch.arange(1000, device="cuda:0")).all())
print("identity ok")
dist.destroy_process_group()
"""
    r = subprocess.run([sys.executable, "-c", code], env=dict(os.environ, PYTHONPATH=ROOT),
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert "identity ok" in r.stdout


def test_unsupported_op_and_overlap_terminate():
    print("[case] pg terminate paths", flush=True)
    pre = """
import torch, torch.distributed as dist
import fairring
from fairring_amd import _fairring
pg = _fairring.ProcessGroup(dist.HashStore(), 0, 1, _fairring.ProcessGroup.Options(50 << 20, 1 << 20, 16))
"""
    env = dict(os.environ, PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, "-c", pre + """
o = dist.AllreduceOptions(); o.reduceOp = dist.ReduceOp.PRODUCT
pg.allreduce([torch.zeros(4, device="cuda:0")], o)
print("survived")
"""], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode != 0 and "survived" not in r.stdout
    assert "ReduceOp::SUM" in r.stderr
    r = subprocess.run([sys.executable, "-c", pre + """
pg.allreduce([torch.zeros(8, device="cuda:0")[::2]])
print("survived")
"""], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode != 0 and "is_non_overlapping_and_dense" in r.stderr


@pytest.mark.parametrize("rank,size", [(0, 2), (3, 8), (6, 7)])
def test_reduce_scatter_base_and_list_form(rank, size):
    # server-side sum with a separate output (fairring/process_group.cc:283-364)
    print("[case] pg reduce_scatter", rank, size, flush=True)
    n = 70_003
    rng = np.random.default_rng(rank * 10 + size)
    x = (rng.standard_normal((size, size * n)) * 0.01).astype(np.float32)   # x[r] = rank r's input
    want = oracle.sum_f32([x[r][rank * n:(rank + 1) * n] for r in range(size)])
    pg = make_pg(rank, size)
    full_in = torch.from_numpy(x[rank].copy()).to(DEV)
    out = torch.empty(n, device=DEV)
    # peers hand in their whole flat inputs
    pg._set_simulated_peer_contributions(
        [torch.from_numpy(x[r].copy()).to(DEV) for r in range(size) if r != rank])
    w = pg._reduce_scatter_base(out, full_in)
    assert w.wait() is True
    torch.cuda.synchronize()
    assert_bits_equal(out.cpu().numpy(), want)
    assert_bits_equal(full_in.cpu().numpy(), x[rank])          # the input is left alone
    # list form, peers hand in just the chunk meant for this rank
    pg._set_simulated_peer_contributions(
        [torch.from_numpy(x[r][rank * n:(rank + 1) * n].copy()).to(DEV)
         for r in range(size) if r != rank])
    out2 = torch.empty(n, device=DEV)
    chunks = list(full_in.view(size, n).unbind(0))
    pg.reduce_scatter([out2], [chunks]).wait()
    torch.cuda.synchronize()
    assert_bits_equal(out2.cpu().numpy(), want)


def test_reduce_scatter_tensor_through_torch_distributed_world_one():
    print("[case] reduce_scatter_tensor world 1", flush=True)
    code = """
import torch, torch.distributed as dist
import fairring
dist.init_process_group("fairring", store=dist.HashStore(), rank=0, world_size=1)
x = torch.arange(1000, dtype=torch.float32, device="cuda:0")
out = torch.empty(1000, device="cuda:0")
dist.reduce_scatter_tensor(out, x)
torch.cuda.synchronize()
assert bool((out == x).all())
print("copy ok")
dist.destroy_process_group()
"""
    r = subprocess.run([sys.executable, "-c", code], env=dict(os.environ, PYTHONPATH=ROOT),
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert "copy ok" in r.stdout
