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


def test_future_asked_for_late_or_twice_or_never():
    """The work waits through the pipeline's own handle; the future is made by
    the first get_future(), also when the operation has long been enqueued, and
    orders its consumers after the reduction all the same."""
    print("[case] pg future made on demand", flush=True)
    size, rank, n = 8, 1, 2_000_003
    rng = np.random.default_rng(15)
    x = (rng.standard_normal((size, n)) * 0.01).astype(np.float32)
    want = oracle.sum_f32(list(x))
    pg = make_pg(rank, size)
    pg._set_simulated_peer_contributions(
        [torch.from_numpy(x[r].copy()).to(DEV) for r in range(size) if r != rank])

    # never: wait() alone orders the current stream after the result
    own = torch.from_numpy(x[rank].copy()).to(DEV)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        side.wait_stream(torch.cuda.default_stream())
        work = pg.allreduce([own])
        assert work.wait() is True
        twice = own * 2          # on `side`, after the reduction
    side.synchronize()
    assert_bits_equal(twice.cpu().numpy(), want * np.float32(2))
    assert work.is_completed() and work.is_success()

    # a small operation goes to the caller's stream; a wait on another stream
    # orders that one after it, and so does the future
    ns = 50_001
    small_want = oracle.sum_f32([r[:ns] for r in x])
    pg._set_simulated_peer_contributions(
        [torch.from_numpy(x[r, :ns].copy()).to(DEV) for r in range(size) if r != rank])
    own = torch.from_numpy(x[rank, :ns].copy()).to(DEV)
    ballast = torch.zeros(64 * MiB, device=DEV)
    pg._synchronize()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        for _ in range(20):
            ballast.add_(1.0)           # the operation queues up behind this
        work = pg.allreduce([own])
    work.wait()                         # the default stream waits for `side`'s operation
    plus = own + 1
    fut = work.get_future()
    other = torch.cuda.Stream()
    with torch.cuda.stream(other):
        times = fut.then(lambda f: f.value()[0] * 3).wait()
    torch.cuda.synchronize()
    assert_bits_equal(own.cpu().numpy(), small_want)
    assert_bits_equal(plus.cpu().numpy(), small_want + np.float32(1))
    assert_bits_equal(times.cpu().numpy(), small_want * np.float32(3))
    pg._set_simulated_peer_contributions(
        [torch.from_numpy(x[r].copy()).to(DEV) for r in range(size) if r != rank])

    # late: the operation is enqueued and finished before anyone asks
    own = torch.from_numpy(x[rank].copy()).to(DEV)
    work = pg.allreduce([own])
    work.wait()
    torch.cuda.synchronize()
    fut = work.get_future()
    assert fut.done()
    assert work.get_future() is fut or work.get_future().done()
    got = fut.then(lambda f: f.value()[0] + 1).wait()
    torch.cuda.synchronize()
    assert fut.value()[0].data_ptr() == own.data_ptr()
    assert_bits_equal(own.cpu().numpy(), want)
    assert_bits_equal(got.cpu().numpy(), want + np.float32(1))

    # at once, then dropped together with the work: the callback still runs
    seen = []
    for i in range(20):
        own = torch.from_numpy(x[rank].copy()).to(DEV)
        pg.allreduce([own]).get_future().then(lambda f, i=i: seen.append(i))
        del own
    pg._synchronize()
    torch.cuda.synchronize()
    assert sorted(seen) == list(range(20))


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


def test_pinned_peers_are_switched_off_by_default():
    print("[case] pg pinned peers refused", flush=True)
    pg = make_pg(0, 2)
    pg._set_simulated_peer_contributions([torch.zeros(100).pin_memory()])
    with pytest.raises(RuntimeError, match="switched off"):
        pg.allreduce([torch.zeros(100, device=DEV)])


@pytest.mark.skip(reason="went silent for 180 s on one GPU run (killed by the harness, GPU still "
                         "answering) after passing on every earlier run; no cause found by reading "
                         "the code or on the CPU stand-in, so the case stays off the GPU and the process group refuses "
                         "pinned peers unless FAIRRING_PINNED_PEERS is set. The same staging "
                         "through the C ABI runs in test_gpu_parity.py and "
                         "test_gpu_random_matrix.py.")
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


def test_group_destroyed_while_python_callbacks_are_pending():
    # the group's destructor drains the command thread, whose completion callbacks run Python
    # code here (future.then): it must not hold the GIL while it waits for them
    print("[case] pg destroyed with callbacks pending", flush=True)
    n = 1 << 20
    pg = make_pg(0, 2)
    own = torch.ones(n, device=DEV)
    pg._set_simulated_peer_contributions([torch.ones(n, device=DEV)])
    seen = []
    futs = [pg.allreduce([own]).get_future().then(lambda f: seen.append(f.value()[0].numel()))
            for _ in range(40)]
    del pg
    for f in futs:
        f.wait()
    torch.cuda.synchronize()
    assert seen == [n] * 40
    assert float(own[0]) == 41.0 and float(own[-1]) == 41.0   # 1, plus the peer's 1 forty times


def test_result_and_synchronize_wait_without_holding_the_interpreter_lock():
    # Python's bindings of Work.result() and Work.synchronize() keep the global lock (those of
    # Work.wait() and Future.wait() let go of it). The completion callback on the command thread
    # needs that lock here (a Python `then` callback; the last reference to a tensor Python made),
    # so a wait inside result() that held on to it would stop both threads for good.
    print("[case] pg result() with Python callbacks pending", flush=True)
    import warnings
    n = 1 << 22
    pg = make_pg(0, 2)
    seen = []
    for i in range(20):
        own = torch.full((n,), float(i), device=DEV)
        pg._set_simulated_peer_contributions([torch.ones(n, device=DEV)])
        work = pg.allreduce([own])
        fut = work.get_future().then(lambda f, i=i: seen.append((i, float(f.value()[0][0]))))
        del own                                  # the future's value holds the last reference
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            if i % 2:
                res = work.result()              # binding keeps the lock while it waits
                assert float(res[0][-1]) == float(i) + 1.0
            else:
                work.synchronize()
        fut.wait()
    torch.cuda.synchronize()
    assert seen == [(i, float(i) + 1.0) for i in range(20)]


def test_data_moving_collectives_exist_for_a_group_of_one_only():
    print("[case] pg broadcast/allgather/barrier", flush=True)
    pg = make_pg(0, 1)
    x = torch.arange(1000, dtype=torch.float32, device=DEV)
    w = pg.broadcast([x])
    assert w.wait() and w.is_completed() and w.result()[0].data_ptr() == x.data_ptr()
    out = torch.zeros(1000, device=DEV)
    pg.allgather([[out]], [x]).wait()
    torch.cuda.synchronize()
    assert bool(torch.equal(out, x))
    out2 = torch.zeros(2, 500, device=DEV)
    pg._allgather_base(out2, x).wait()
    torch.cuda.synchronize()
    assert bool(torch.equal(out2.reshape(-1), x))
    assert pg.barrier().wait()
    pg2 = make_pg(0, 2)
    for call in (lambda: pg2.broadcast([x]), lambda: pg2.allgather([[out, out]], [x]),
                 lambda: pg2._allgather_base(torch.zeros(2000, device=DEV), x), pg2.barrier):
        with pytest.raises(RuntimeError, match="needs a transport"):
            call()


def test_allreduce_from_two_threads_and_futures_with_callbacks():
    # two threads share the group (its submit path is serialised inside); each reduces its
    # own tensors 30 times and chains a Python callback on every future, which the command
    # thread runs: no result may be lost, late or mixed up
    import threading
    print("[case] pg two threads", flush=True)
    size, rank, n = 4, 1, 200_003
    pg = make_pg(rank, size, slice_bytes=256 * 1024, total=MiB)
    gen = torch.Generator(device=DEV)
    gen.manual_seed(91)
    peers = [torch.randn(n, device=DEV, generator=gen) * 0.01 for _ in range(size - 1)]
    pg._set_simulated_peer_contributions(peers)
    torch.cuda.synchronize()
    failures, seen = [], []

    def worker(tid):
        try:
            g = torch.Generator(device=DEV)
            g.manual_seed(92 + tid)
            for i in range(30):
                own = torch.randn(n, device=DEV, generator=g) * 0.01
                chain = ordered(own.clone(), peers, rank)
                want = chain[0].clone()
                for c in chain[1:]:
                    want += c
                fut = pg.allreduce([own]).get_future().then(
                    lambda f, tag=(tid, i): (seen.append(tag), f.value()[0])[1])
                got = fut.wait()
                torch.cuda.current_stream().synchronize()
                if got.data_ptr() != own.data_ptr() or not bool(
                        torch.equal(got.view(torch.int32), want.view(torch.int32))):
                    failures.append("thread %d op %d" % (tid, i))
        except Exception as e:  # noqa: BLE001
            failures.append("thread %d: %r" % (tid, e))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a thread did not finish"
    assert not failures, failures[:5]
    assert sorted(seen) == [(t, i) for t in range(2) for i in range(30)]


def test_peers_replaced_while_operations_wait_in_the_queue_stay_alive():
    # The command thread is held inside a completion callback (a Python `then` that waits on a
    # flag) while more operations queue up behind it; the group is then handed new peers, the
    # old ones are dropped and tensors of the same size, full of other values, are allocated at
    # once (the caching allocator hands a freed block straight back). The queued operations must
    # still see the peers they were submitted with.
    print("[case] pg peers replaced under queued operations", flush=True)
    import threading
    n = 1 << 23           # large enough to go through the command thread, not the caller's stream
    pg = make_pg(0, 2)
    warm = torch.ones(n, device=DEV)
    pg._set_simulated_peer_contributions([torch.ones(n, device=DEV)])
    pg.allreduce([warm]).wait()
    torch.cuda.synchronize()
    gate = threading.Event()
    first = torch.zeros(n, device=DEV)
    pg._set_simulated_peer_contributions([torch.full((n,), 10.0, device=DEV)])
    held = pg.allreduce([first]).get_future().then(lambda f: gate.wait(30))
    owns = [torch.full((n,), float(i), device=DEV) for i in range(1, 5)]
    works = [pg.allreduce([o]) for o in owns]            # queued behind the held thread
    pg._set_simulated_peer_contributions([torch.full((n,), -1.0, device=DEV)])
    junk = [torch.full((n,), 12345.0, device=DEV) for _ in range(4)]   # lands where the old peer was
    torch.cuda.synchronize()
    gate.set()
    held.wait()
    for w in works:
        w.wait()
    torch.cuda.synchronize()
    assert float(first[0]) == 10.0
    for i, o in enumerate(owns, start=1):
        assert float(o.min()) == float(o.max()) == i + 10.0, (i, float(o.min()), float(o.max()))
    del junk


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


# ---- seeded random walk over the process group's surface -------------------------------------

_PG_KINDS = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16,
             "f64": torch.float64, "i32": torch.int32, "i64": torch.int64, "u8": torch.uint8,
             "i8": torch.int8}


def _pg_values(kind, rng, k, n):
    if oracle.TYPES[kind][1]:
        x = rng.standard_normal((k, n)) * np.exp(rng.uniform(-6, 6, (k, n)))
        if kind == "f64":
            return x
        x = x.astype(np.float32)
        if kind == "bf16":
            return oracle.np_f32_to_bf16_rne(x).reshape(k, n)
        if kind == "f16":
            return x.astype(np.float16).view(np.uint16)
        return x
    info = np.iinfo(oracle.TYPES[kind][0])
    return rng.integers(info.min, int(info.max) + 1, (k, n), dtype=oracle.TYPES[kind][0])


def _pg_tensor(a, tdt, pinned=False):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if tdt in (torch.float16, torch.bfloat16):
        t = t.view(torch.int16).view(tdt)
    return t.pin_memory() if pinned else t.to(DEV)


def _pg_bits(t):
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


@pytest.mark.parametrize("seed", range(60))
def test_random_process_group_case(seed):
    import zlib
    rng = np.random.default_rng(zlib.crc32(b"fairring-pg-matrix") + seed)
    kind = list(_PG_KINDS)[rng.integers(len(_PG_KINDS))]
    tdt = _PG_KINDS[kind]
    floating = oracle.TYPES[kind][1]
    size = int(rng.choice([1, 2, 3, 5, 8, 16, 48, 65, 100]))
    rank = int(rng.integers(size))
    op = "max" if rng.random() < 0.25 else "sum"
    form = ["allreduce", "allreduce", "reduce_scatter_base", "pre_divided"][rng.integers(4)]
    if form == "pre_divided" and (not floating or op != "sum"):
        form = "allreduce"
    divide = bool(floating and op == "sum" and form != "pre_divided" and rng.random() < 0.5)
    pinned = False   # peers in pinned host memory are switched off in the process group
    n = int(rng.choice([1, 33, 4099, 100_003]))
    if size > 16:
        n = min(n, 4099)
    slice_bytes = int(rng.choice([16 * 1024, 256 * 1024]))
    case = dict(seed=seed, kind=kind, size=size, rank=rank, op=op, form=form, divide=divide,
                pinned=pinned, n=n, slice_bytes=slice_bytes)
    print("[case] pg random", case, flush=True)
    pg = make_pg(rank, size, total=2 * slice_bytes, slice_bytes=slice_bytes, parallelism=2)
    pg._set_fused_divide(divide)
    ropts = dist.AllreduceOptions() if form != "reduce_scatter_base" else dist.ReduceScatterOptions()
    ropts.reduceOp = dist.ReduceOp.MAX if op == "max" else dist.ReduceOp.SUM
    if form == "reduce_scatter_base":
        x = _pg_values(kind, rng, size, size * n)                    # x[r] = rank r's whole input
        host = [x[r][rank * n:(rank + 1) * n] for r in range(size)]
        pg._set_simulated_peer_contributions(
            [_pg_tensor(x[r], tdt) for r in range(size) if r != rank])
        out = torch.empty(n, dtype=tdt, device=DEV)
        pg._reduce_scatter_base(out, _pg_tensor(x[rank], tdt), ropts).wait()
    else:
        x = _pg_values(kind, rng, size, n)
        host = list(x)
        pg._set_simulated_peer_contributions(
            [_pg_tensor(x[r], tdt, pinned) for r in range(size) if r != rank])
        out = _pg_tensor(x[rank], tdt)
        if form == "pre_divided":
            pg._allreduce_pre_divided(out).wait()
        else:
            pg.allreduce([out], ropts).wait()
    torch.cuda.synchronize()
    pow2 = size & (size - 1) == 0
    if form == "pre_divided":
        want = oracle.reduce(kind, host, "sum", oracle.SCALE_PRE_MUL,
                             float(np.float32(1) / np.float32(size)))
    elif divide and size > 1:
        want = oracle.reduce(kind, host, "sum", oracle.SCALE_MUL if pow2 else oracle.SCALE_DIV,
                             1.0 / size if pow2 else float(size))
    else:
        want = oracle.reduce(kind, host, op)
    got = _pg_bits(out)
    if op == "max" and floating:    # the sign of a zero maximum is not specified
        zero = (want == 0) if kind in ("f32", "f64") else ((want & 0x7FFF) == 0)
        got, want = got[~zero], want[~zero]
    assert_bits_equal(got, want, str(case), half=kind == "f16")


@pytest.mark.parametrize("consumer", ["default", "side"])
def test_waiting_on_every_bucket_orders_the_consumer_after_all_of_them(consumer):
    """DDP's end of backward: every bucket's work is waited for on one stream,
    which then reads the results with no host synchronisation in between. On
    the default (null) stream the pipeline tells that stream only once per
    reduce stream what to wait for; the results must be complete all the same."""
    print("[case] pg waits on every bucket, consumer on the", consumer, "stream", flush=True)
    size, rank, nb, n = 4, 1, 24, 16 * MiB          # 24 buckets of 64 MiB
    g = torch.Generator(device=DEV)
    g.manual_seed(33)
    peers = [torch.empty(n, device=DEV).normal_(0, 1.0, generator=g) for _ in range(size - 1)]
    owns = [torch.empty(n, device=DEV).normal_(0, 1.0, generator=g) for _ in range(nb)]
    want = []
    for o in owns:                                   # rank order: peer 0, own, peers 1 and 2
        acc = peers[0] + o
        acc.add_(peers[1]).add_(peers[2])
        want.append(acc)
    pg = make_pg(rank, size, slice_bytes=25 * MiB)
    pg._set_simulated_peer_contributions(peers)
    stream = torch.cuda.default_stream() if consumer == "default" else torch.cuda.Stream()
    with torch.cuda.stream(stream):                  # the comparison's kernels loaded beforehand:
        torch.equal(want[0].view(torch.int32), want[1].view(torch.int32))   # the first call takes 0.1 s
    torch.cuda.synchronize()
    works = [pg.allreduce([o]) for o in owns]        # 7.7 GB of traffic: still running below
    with torch.cuda.stream(stream):
        for w in works:
            assert w.wait() is True
        # reads on `stream`, right behind the waits; the bucket submitted last first,
        # which is the one still furthest from done
        same = [torch.equal(o.view(torch.int32), w_.view(torch.int32))
                for o, w_ in zip(reversed(owns), reversed(want))]
    assert all(same)
    pg._synchronize()
    torch.cuda.synchronize()


def test_collectives_issued_back_to_back_on_one_tensor_run_in_order():
    """No wait between them, as with any c10d backend. An in-place allreduce of
    a 64 MiB tensor is followed at once by one of its last quarter (which would
    otherwise start on the other reduce stream while the first is still at the
    front of the tensor), three times over; then a reduce-scatter whose output's
    tail is allreduced at once."""
    print("[case] pg back-to-back collectives on one tensor", flush=True)
    size, rank, n = 4, 1, 16 * MiB
    m = n // 4
    g = torch.Generator(device=DEV)
    g.manual_seed(44)
    peers = [torch.empty(n, device=DEV).normal_(0, 0.01, generator=g) for _ in range(size - 1)]
    tails = [p[n - m:] for p in peers]
    own = torch.empty(n, device=DEV).normal_(0, 0.01, generator=g)
    start = own.clone()
    pg = make_pg(rank, size, slice_bytes=25 * MiB)
    pg._set_simulated_peer_contributions(peers)
    warm = torch.zeros(n, device=DEV)
    pg.allreduce([warm]).wait()                       # the first launch loads the code object
    torch.cuda.synchronize()

    def fold(mine, others):                           # rank order: peer 0, this rank, peers 1 and 2
        acc = others[0] + mine
        return acc.add_(others[1]).add_(others[2])

    works = []
    for _ in range(3):
        pg._set_simulated_peer_contributions(peers)
        works.append(pg.allreduce([own]))
        pg._set_simulated_peer_contributions(tails)
        works.append(pg.allreduce([own[n - m:]]))
    for w in works:
        w.wait()
    torch.cuda.synchronize()
    want = start
    for _ in range(3):
        want = fold(want, peers)
        want[n - m:] = fold(want[n - m:], tails)
    assert bool(torch.equal(own.view(torch.int32), want.view(torch.int32)))

    whole = torch.empty(size * n, device=DEV).normal_(0, 0.01, generator=g)
    out = torch.zeros(n, device=DEV)
    torch.cuda.synchronize()
    pg._set_simulated_peer_contributions(peers)
    w1 = pg._reduce_scatter_base(out, whole, dist.ReduceScatterOptions())
    pg._set_simulated_peer_contributions(tails)
    w2 = pg.allreduce([out[n - m:]])
    w1.wait()
    w2.wait()
    torch.cuda.synchronize()
    want = fold(whole[rank * n:(rank + 1) * n], peers)
    want[n - m:] = fold(want[n - m:], tails)
    assert bool(torch.equal(out.view(torch.int32), want.view(torch.int32)))
    pg._synchronize()
