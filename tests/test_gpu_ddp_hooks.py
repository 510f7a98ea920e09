"""GPU tests of the DDP communication hooks of the "fairring" backend: the
process group's hooked allreduce entry points and fairring_amd.ddp_comm_hooks
against the CPU oracle, and against torch's own hooks
(torch:distributed/algorithms/ddp_comm_hooks/default_hooks.py) in a real DDP
backward pass."""
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
from fairring_amd import _fairring, ddp_comm_hooks  # noqa: E402

DEV = "cuda:0"
MiB = 1024 * 1024
WIRES = [("bf16", torch.bfloat16), ("f16", torch.float16)]


def make_pg(rank, size, total=MiB, slice_bytes=256 * 1024):
    o = _fairring.ProcessGroup.Options(
        max_memory_allocated_in_bytes=total, max_padding_allocated_in_bytes=MiB,
        min_parallelism=2, is_high_priority_stream=True,
        timeout=datetime.timedelta(seconds=60), slice_size_in_bytes=slice_bytes)
    return _fairring.ProcessGroup(dist.HashStore(), rank, size, o)


class Bucket:
    """What a hook reads of a dist.GradBucket."""

    def __init__(self, t):
        self._t = t

    def buffer(self):
        return self._t


def bits16(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("rank,size", [(0, 2), (2, 6), (7, 8), (11, 48)])
def test_pre_divided_allreduce(rank, size):
    print("[case] pg pre-divided", rank, size, flush=True)
    n = 300_007
    rng = np.random.default_rng(900 + size)
    x = (rng.standard_normal((size, n)) * 0.01).astype(np.float32)
    pg = make_pg(rank, size)
    own = torch.from_numpy(x[rank].copy()).to(DEV)
    pg._set_simulated_peer_contributions(
        [torch.from_numpy(x[r].copy()).to(DEV) for r in range(size) if r != rank])
    fut = ddp_comm_hooks.allreduce_hook(pg, Bucket(own))
    got = fut.wait()
    torch.cuda.synchronize()
    assert got.data_ptr() == own.data_ptr()
    s = float(np.float32(1) / np.float32(size))
    assert_bits_equal(own.cpu().numpy(), oracle.sum_f32(list(x), oracle.SCALE_PRE_MUL, s))


@pytest.mark.parametrize("wire,tdt", WIRES)
@pytest.mark.parametrize("rank,size", [(0, 3), (3, 8), (16, 17)])
def test_compressed_allreduce(wire, tdt, rank, size):
    print("[case] pg compressed", wire, rank, size, flush=True)
    n = 300_007
    rng = np.random.default_rng(950 + size)
    x = (rng.standard_normal((size, n)) * 0.01).astype(np.float32)
    pg = make_pg(rank, size)
    own = torch.from_numpy(x[rank].copy()).to(DEV)
    # what the other ranks' hooks leave in their compressed tensors
    comp = [torch.from_numpy(x[r].copy()).to(tdt).div_(size) for r in range(size)]
    pg._set_simulated_peer_contributions([comp[r].to(DEV) for r in range(size) if r != rank])
    hook = ddp_comm_hooks.bf16_compress_hook if wire == "bf16" else ddp_comm_hooks.fp16_compress_hook
    got = hook(pg, Bucket(own)).wait()
    torch.cuda.synchronize()
    assert got.data_ptr() == own.data_ptr() and got.dtype == torch.float32
    contribs = [bits16(c) for c in comp]
    contribs[rank] = x[rank]
    s = float(np.float32(1) / np.float32(size))
    assert_bits_equal(own.cpu().numpy(),
                      oracle.compressed_sum(contribs, rank, wire, oracle.SCALE_MUL, s))


class GradBucket(Bucket):
    """A bucket with the parameters it was assembled from."""

    def __init__(self, t, params):
        super().__init__(t)
        self._params = params

    def parameters(self):
        return self._params

    def gradients(self):
        views, off = [], 0
        for p in self._params:
            views.append(self._t[off:off + p.numel()].view_as(p))
            off += p.numel()
        return views


@pytest.mark.parametrize("kind,tdt", [("f32", torch.float32), ("bf16", torch.bfloat16)])
@pytest.mark.parametrize("rank,size", [(0, 2), (5, 8), (2, 3)])
def test_allreduce_from_grads(kind, tdt, rank, size):
    # the bucket's own contribution is read from the gradient tensors; the bucket itself holds
    # garbage on the way in
    print("[case] pg from grads", kind, rank, size, flush=True)
    shapes = [(1024, 512), (512,), (1,), (300, 7), (64, 64, 3), (5,)]
    n = sum(int(np.prod(sh)) for sh in shapes)
    rng = np.random.default_rng(40 * size + rank)
    x = (rng.standard_normal((size, n)) * 0.01).astype(np.float32)
    if kind == "bf16":
        bits = oracle.np_f32_to_bf16_rne(x)
        host = list(bits)
        dev_of = lambda a: torch.from_numpy(a.view(np.int16).copy()).to(DEV).view(tdt)  # noqa: E731
    else:
        host = list(x)
        dev_of = lambda a: torch.from_numpy(a.copy()).to(DEV)  # noqa: E731
    pg = make_pg(rank, size)
    pg._set_simulated_peer_contributions([dev_of(host[r]) for r in range(size) if r != rank])
    grads, off = [], 0
    for sh in shapes:
        ln = int(np.prod(sh))
        grads.append(dev_of(host[rank][off:off + ln]).view(sh))
        off += ln
    s = float(np.float32(1) / np.float32(size))
    for pre in (True, False):
        bucket = torch.full((n,), float("nan"), dtype=tdt, device=DEV)
        work = pg._allreduce_from_grads(bucket, grads, pre)
        work.wait()
        torch.cuda.synchronize()
        want = oracle.reduce(kind, host, "sum", oracle.SCALE_PRE_MUL if pre else oracle.SCALE_NONE, s)
        got = bucket.cpu().numpy() if kind == "f32" else bits16(bucket)
        assert_bits_equal(got, want, "%s pre=%s" % (kind, pre))
    # the hook: same bits as allreduce_hook on a bucket the gradients were copied into
    params = []
    for gr in grads:
        p = torch.nn.Parameter(torch.zeros_like(gr))
        p.grad = gr
        params.append(p)
    bucket = torch.cat([gr.reshape(-1) for gr in grads])
    via_hook = ddp_comm_hooks.allreduce_from_grads_hook(pg, GradBucket(bucket.clone().fill_(7), params))
    got = via_hook.wait()
    torch.cuda.synchronize()
    want = ddp_comm_hooks.allreduce_hook(pg, Bucket(bucket)).wait()
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16 if kind == "bf16" else torch.int32),
                       want.view(torch.int16 if kind == "bf16" else torch.int32))
    with pytest.raises(RuntimeError, match="gradients hold"):
        pg._allreduce_from_grads(bucket, grads[:-1], True)


@pytest.mark.parametrize("wire,tdt", [("bf16", torch.bfloat16), ("f16", torch.float16)])
@pytest.mark.parametrize("rank,size", [(0, 2), (5, 8), (2, 3)])
def test_allreduce_compressed_from_grads(wire, tdt, rank, size):
    # the compression hooks' reduction with the bucket's own fp32 contribution read from the
    # gradient tensors: the bucket holds garbage on the way in and the oracle's result on the
    # way out, and the hook gives the bits of the hook that reads an assembled bucket
    print("[case] pg compressed from grads", wire, rank, size, flush=True)
    shapes = [(1024, 512), (512,), (1,), (300, 7), (64, 64, 3), (5,)]
    n = sum(int(np.prod(sh)) for sh in shapes)
    rng = np.random.default_rng(50 * size + rank)
    x = (rng.standard_normal((size, n)) * 0.01).astype(np.float32)
    bits = oracle.np_f32_to_bf16_rne(x) if wire == "bf16" else x.astype(np.float16).view(np.uint16)
    pg = make_pg(rank, size)
    pg._set_simulated_peer_contributions(
        [torch.from_numpy(bits[r].view(np.int16).copy()).to(DEV).view(tdt)
         for r in range(size) if r != rank])
    grads, off = [], 0
    for sh in shapes:
        ln = int(np.prod(sh))
        grads.append(torch.from_numpy(x[rank, off:off + ln].copy()).to(DEV).view(sh))
        off += ln
    bucket = torch.full((n,), float("nan"), device=DEV)
    pg._allreduce_compressed(bucket, tdt, grads).wait()
    torch.cuda.synchronize()
    contribs = [bits[r] for r in range(size)]
    contribs[rank] = x[rank]
    s = float(np.float32(1) / np.float32(size))
    assert_bits_equal(bucket.cpu().numpy(),
                      oracle.compressed_sum(contribs, rank, wire, oracle.SCALE_MUL, s))
    params = []
    for gr in grads:
        p = torch.nn.Parameter(torch.zeros_like(gr))
        p.grad = gr
        params.append(p)
    assembled = torch.cat([gr.reshape(-1) for gr in grads])
    hook = getattr(ddp_comm_hooks, "%s_compress_from_grads_hook" % ("bf16" if wire == "bf16" else "fp16"))
    plain = getattr(ddp_comm_hooks, "%s_compress_hook" % ("bf16" if wire == "bf16" else "fp16"))
    got = hook(pg, GradBucket(assembled.clone().fill_(7), params)).wait()
    torch.cuda.synchronize()
    want = plain(pg, Bucket(assembled)).wait()
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    with pytest.raises(RuntimeError, match="gradients hold"):
        pg._allreduce_compressed(bucket, tdt, grads[:-1])


def test_hook_contract_errors():
    print("[case] pg hook errors", flush=True)
    pg = make_pg(0, 2)
    own = torch.zeros(100, device=DEV)
    with pytest.raises(RuntimeError, match="simulated peer"):
        pg._allreduce_compressed(own, torch.bfloat16)
    pg._set_simulated_peer_contributions([torch.zeros(100, device=DEV)])
    with pytest.raises(RuntimeError, match="elements of"):          # peer not in the wire type
        pg._allreduce_compressed(own, torch.bfloat16)
    with pytest.raises(RuntimeError, match="float32 bucket"):
        pg._allreduce_compressed(own.half(), torch.float16)
    with pytest.raises(RuntimeError, match="wire type"):
        pg._allreduce_compressed(own, torch.float64)
    pg._set_simulated_peer_contributions([torch.zeros(100, dtype=torch.int32, device=DEV)])
    with pytest.raises(RuntimeError, match="floating-point"):
        pg._allreduce_pre_divided(torch.zeros(100, dtype=torch.int32, device=DEV))
    with pytest.raises(RuntimeError, match="'fairring' backend"):
        ddp_comm_hooks.bf16_compress_hook(object(), Bucket(own))


DDP_SCRIPT = """
import torch, torch.distributed as dist
import torch.nn as nn
from torch.nn.parallel import DistributedDataParallel as DDP
from torch.distributed.algorithms.ddp_comm_hooks import default_hooks as torch_hooks
import fairring
from fairring_amd import ddp_comm_hooks as ours

dist.init_process_group("fairring", store=dist.HashStore(), rank=0, world_size=1)

def grads(hook):
    torch.manual_seed(0)
    model = nn.Sequential(nn.Linear(512, 1024), nn.GELU(), nn.Linear(1024, 1024), nn.GELU(),
                          nn.Linear(1024, 10)).to("cuda:0")
    ddp = DDP(model, device_ids=[0], bucket_cap_mb=1)   # init_sync: broadcast + allgather, group of one
    if hook is not None:
        ddp.register_comm_hook(None, hook)
    x = torch.randn(64, 512, device="cuda:0", generator=torch.Generator("cuda:0").manual_seed(1))
    ddp(x).square().mean().backward()
    torch.cuda.synchronize()
    return [p.grad.clone() for p in model.parameters()]

plain = grads(None)
for name in ("allreduce_hook", "bf16_compress_hook", "fp16_compress_hook"):
    want = grads(getattr(torch_hooks, name))
    got = grads(getattr(ours, name))
    for a, b in zip(want, got):
        assert a.dtype == b.dtype == torch.float32
        assert torch.equal(a.view(torch.int32), b.view(torch.int32)), name
    print(name, "ok", flush=True)
for a, b in zip(plain, grads(ours.allreduce_hook)):
    assert torch.equal(a.view(torch.int32), b.view(torch.int32))
# gradient_as_bucket_view=False is DDP's default, used above: the hook that reads the gradients
# where autograd left them gives the bits of torch's allreduce_hook
for a, b in zip(grads(torch_hooks.allreduce_hook), grads(ours.allreduce_from_grads_hook)):
    assert torch.equal(a.view(torch.int32), b.view(torch.int32))
print("allreduce_from_grads_hook ok", flush=True)
for name in ("bf16_compress", "fp16_compress"):
    want = grads(getattr(torch_hooks, name + "_hook"))
    got = grads(getattr(ours, name + "_from_grads_hook"))
    for a, b in zip(want, got):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32)), name
    print(name + "_from_grads_hook ok", flush=True)
print("ddp hooks ok")
dist.destroy_process_group()
"""


def test_hooks_in_a_ddp_backward_pass_equal_torchs_own():
    # world size 1 (one GPU, no transport): the hooks still cast, divide and copy back, and
    # DDP drives them bucket by bucket from its autograd hooks
    print("[case] ddp backward with hooks", flush=True)
    r = subprocess.run([sys.executable, "-c", DDP_SCRIPT], env=dict(os.environ, PYTHONPATH=ROOT),
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
    assert "ddp hooks ok" in r.stdout
