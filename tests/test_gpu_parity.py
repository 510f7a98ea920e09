"""GPU parity: the HIP kernels and the slice pipeline, called through the C ABI,
against the CPU oracle and the committed golden vectors. Bit-exact for fp32 and
for bf16 (the contract allows 1 bf16 ulp; the kernel meets 0).
"""
import zlib

import numpy as np
import pytest
import torch

import oracle
from conftest import assert_bits_equal

pytestmark = pytest.mark.gpu

fa = pytest.importorskip("fairring_amd")

DEV = "cuda:0"
MiB = 1024 * 1024


def _print_case(*a):
    print("[case]", *a, flush=True)


def to_gpu_f32(x):
    return [torch.from_numpy(np.ascontiguousarray(r)).to(DEV) for r in x]


def to_gpu_bf16(bits):
    return [torch.from_numpy(np.ascontiguousarray(r).view(np.int16)).to(DEV).view(torch.bfloat16)
            for r in bits]


def bf16_bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


F32_CASES = ["f32_k2", "f32_k3", "f32_k8", "f32_k17", "f32_k64"]
BF16_CASES = ["bf16_k2", "bf16_k8", "bf16_k64"]
MODES = [("sum", fa.SCALE_NONE, None), ("mul", fa.SCALE_MUL, "inv"), ("div", fa.SCALE_DIV, "k")]


@pytest.mark.parametrize("case", F32_CASES)
def test_kernel_f32_golden(golden, case):
    x = golden[case + "_in"]
    k = x.shape[0]
    xs = to_gpu_f32(x)
    for name, mode, s in MODES:
        _print_case("golden", case, name)
        scale = 1.0 if s is None else (1.0 / k if s == "inv" else float(k))
        out = torch.empty_like(xs[0])
        fa.reduce_slice(out, xs, scale_mode=mode, scale=scale)
        torch.cuda.synchronize()
        assert_bits_equal(out.cpu().numpy(), golden[case + "_" + name], case + " " + name)


@pytest.mark.parametrize("case", BF16_CASES)
def test_kernel_bf16_golden(golden, case):
    x = golden[case + "_in"]
    k = x.shape[0]
    xs = to_gpu_bf16(x)
    for name, mode, s in MODES:
        _print_case("golden", case, name)
        scale = 1.0 if s is None else (1.0 / k if s == "inv" else float(k))
        out = torch.empty_like(xs[0])
        fa.reduce_slice(out, xs, scale_mode=mode, scale=scale)
        torch.cuda.synchronize()
        assert_bits_equal(bf16_bits(out), golden[case + "_" + name], case + " " + name)


@pytest.mark.parametrize("k", [1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 33, 64])
@pytest.mark.parametrize("n", [1, 3, 4, 5, 255, 1024, 4099, 262147])
def test_kernel_f32_vs_oracle_sizes(k, n):
    _print_case("f32 sizes", k, n)
    rng = np.random.default_rng(1000 * k + n)
    x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
    xs = to_gpu_f32(x)
    out = torch.empty_like(xs[0])
    fa.reduce_slice(out, xs, scale_mode=fa.SCALE_DIV, scale=float(k))
    torch.cuda.synchronize()
    assert_bits_equal(out.cpu().numpy(), oracle.sum_f32(list(x), oracle.SCALE_DIV, float(k)))


@pytest.mark.parametrize("k", [1, 2, 3, 8, 13, 64])
@pytest.mark.parametrize("n", [1, 7, 8, 9, 1023, 131075])
def test_kernel_bf16_vs_oracle_sizes(k, n):
    _print_case("bf16 sizes", k, n)
    rng = np.random.default_rng(2000 * k + n)
    x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
    bits = oracle.np_f32_to_bf16_rne(x)
    xs = to_gpu_bf16(bits)
    out = torch.empty_like(xs[0])
    fa.reduce_slice(out, xs, scale_mode=fa.SCALE_MUL, scale=1.0 / k)
    torch.cuda.synchronize()
    assert_bits_equal(bf16_bits(out), oracle.sum_bf16(list(bits), oracle.SCALE_MUL, 1.0 / k))


@pytest.mark.parametrize("head", [0, 1, 2, 3])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_kernel_unaligned_congruent(head, dtype):
    # every pointer shifted by the same number of elements off a 16-byte boundary
    _print_case("unaligned congruent", head, dtype)
    k, n = 8, 10007
    rng = np.random.default_rng(77 + head)
    x = (rng.standard_normal((k, n + head)) * 0.01).astype(np.float32)
    if dtype == "f32":
        big = to_gpu_f32(x)
        outb = torch.zeros(n + head, dtype=torch.float32, device=DEV)
        fa.reduce_slice(outb[head:], [b[head:] for b in big])
        torch.cuda.synchronize()
        assert_bits_equal(outb[head:].cpu().numpy(), oracle.sum_f32(list(x[:, head:])))
        assert (outb[:head] == 0).all()
    else:
        bits = oracle.np_f32_to_bf16_rne(x)
        big = to_gpu_bf16(bits)
        outb = torch.zeros(n + head, dtype=torch.bfloat16, device=DEV)
        fa.reduce_slice(outb[head:], [b[head:] for b in big])
        torch.cuda.synchronize()
        assert_bits_equal(bf16_bits(outb[head:]), oracle.sum_bf16(list(bits[:, head:])))
        assert (outb[:head] == 0).all()


def test_kernel_mismatched_alignment_falls_back():
    _print_case("mismatched alignment")
    k, n = 5, 5003
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((k, n + 4)) * 0.01).astype(np.float32)
    big = to_gpu_f32(x)
    views = [b[(i % 4):(i % 4) + n] for i, b in enumerate(big)]
    out = torch.empty(n, dtype=torch.float32, device=DEV)
    fa.reduce_slice(out, views)
    torch.cuda.synchronize()
    want = oracle.sum_f32([x[i, (i % 4):(i % 4) + n] for i in range(k)])
    assert_bits_equal(out.cpu().numpy(), want)


def test_kernel_in_place_and_carry():
    _print_case("in place / carry")
    k, n = 8, 70001
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
    xs = to_gpu_f32(x)
    want = oracle.sum_f32(list(x), oracle.SCALE_MUL, 0.125)
    # in place into contribution 3's buffer (the reference reduces into its own shard)
    fa.reduce_slice(xs[3], xs, scale_mode=fa.SCALE_MUL, scale=0.125)
    torch.cuda.synchronize()
    assert_bits_equal(xs[3].cpu().numpy(), want)
    # chained launches with carry reproduce the single-launch order
    xs = to_gpu_f32(x)
    out = torch.empty_like(xs[0])
    fa.reduce_slice(out, xs[:3])
    fa.reduce_slice(out, xs[3:5], carry=True)
    fa.reduce_slice(out, xs[5:], carry=True, scale_mode=fa.SCALE_MUL, scale=0.125)
    torch.cuda.synchronize()
    assert_bits_equal(out.cpu().numpy(), want)


def test_kernel_max():
    _print_case("max")
    k, n = 6, 40003
    rng = np.random.default_rng(8)
    x = rng.standard_normal((k, n)).astype(np.float32)
    x[2, 5] = np.nan
    xs = to_gpu_f32(x)
    out = torch.empty_like(xs[0])
    fa.reduce_slice(out, xs, op=fa.MAX)
    torch.cuda.synchronize()
    assert_bits_equal(out.cpu().numpy(), oracle.max_f32(list(x)))
    bits = oracle.np_f32_to_bf16_rne(x)
    xb = to_gpu_bf16(bits)
    outb = torch.empty_like(xb[0])
    fa.reduce_slice(outb, xb, op=fa.MAX)
    torch.cuda.synchronize()
    assert_bits_equal(bf16_bits(outb), oracle.max_bf16(list(bits)))


@pytest.mark.parametrize("k", [2, 8, 64])
def test_reference_known_answers(k):
    # benchmark/benchmark.cc:130-186: all ones -> world size; arange -> arange * world
    _print_case("KAT", k)
    n = 6_553_600 if k <= 8 else 262_144
    ones = torch.ones(n, device=DEV)
    out = torch.empty_like(ones)
    fa.reduce_slice(out, [ones] * k)
    torch.cuda.synchronize()
    assert bool((out == float(k)).all())
    m = min(n, (1 << 24) // k)
    ar = torch.arange(m, dtype=torch.float32, device=DEV)
    out = torch.empty_like(ar)
    fa.reduce_slice(out, [ar] * k)
    torch.cuda.synchronize()
    assert bool((out == ar * k).all())


def test_error_paths():
    _print_case("errors")
    a = torch.zeros(1000, device=DEV)
    with pytest.raises(fa.FairringError):  # partial overlap of output and input
        fa.reduce_slice(a[0:600], [a[100:700], a[0:600]])
    with pytest.raises(fa.FairringError):  # unsupported dtype
        fa.reduce_slice(a.to(torch.int16), [a.to(torch.int16)])
    with pytest.raises(fa.FairringError):  # K beyond one launch
        fa.reduce_slice(a, [a] * 65)
    with pytest.raises(fa.FairringError):  # MAX with a scale
        fa.reduce_slice(a, [a, a], op=fa.MAX, scale_mode=fa.SCALE_MUL, scale=0.5)
    empty = torch.zeros(0, device=DEV)
    fa.reduce_slice(empty, [empty, empty])  # empty is a no-op, not an error
    torch.cuda.synchronize()


# ---- pipeline -----------------------------------------------------------------------

@pytest.mark.parametrize("slice_bytes,total,streams", [
    (4096, 8192, 0), (40000, 400000, 3), (25 * MiB, 50 * MiB, 0), (0, 50 * MiB, 0)])
def test_pipeline_resident_independent_of_slicing(slice_bytes, total, streams):
    _print_case("pipeline resident", slice_bytes, total, streams)
    k, n = 8, 300_007
    rng = np.random.default_rng(31)
    x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
    xs = to_gpu_f32(x)
    out = torch.empty_like(xs[0])
    dev = fa.DeviceFairring(0, max_memory_allocated_in_bytes=total,
                            slice_size_in_bytes=slice_bytes, num_reduce_streams=streams)
    w = dev.allreduce(out, xs, scale_mode=fa.SCALE_MUL, scale=0.125)
    assert w.wait() is True and w.is_completed()
    assert_bits_equal(out.cpu().numpy(), oracle.sum_f32(list(x), oracle.SCALE_MUL, 0.125))
    # stream-ordered consumption without a host wait
    out2 = torch.empty_like(xs[0])
    w2 = dev.allreduce(out2, xs)
    w2.block_stream()
    doubled = out2 * 2
    torch.cuda.synchronize()
    want = oracle.sum_f32(list(x))
    assert_bits_equal(doubled.cpu().numpy(), want * np.float32(2))
    dev.close()


def test_block_stream_orders_a_consumer_behind_a_long_operation():
    # hundreds of launches over three streams are still in flight when the consumer is enqueued
    # on the caller's stream right behind block_stream(): it must see the finished result
    _print_case("block_stream, long operation")
    k, n = 8, 100_000_007
    g = torch.Generator(device=DEV)
    g.manual_seed(77)
    xs = [torch.empty(n, device=DEV).normal_(0, 0.01, generator=g) for _ in range(k)]
    out = torch.zeros(n, device=DEV)
    dev = fa.DeviceFairring(0, slice_size_in_bytes=4 * MiB, max_memory_allocated_in_bytes=8 * MiB,
                            num_reduce_streams=3, max_launch_bytes=MiB)
    torch.cuda.synchronize()
    w = dev.allreduce(out, xs, scale_mode=fa.SCALE_MUL, scale=0.125)
    w.block_stream()
    doubled = out * 2           # on torch's current stream, no host wait in between
    nonzero = int(torch.count_nonzero(doubled))
    w.wait()
    chain = xs[0].clone()
    for x in xs[1:]:
        chain.add_(x)
    chain.mul_(0.125)
    assert bool(torch.equal(out.view(torch.int32), chain.view(torch.int32)))
    assert bool(torch.equal(doubled.view(torch.int32), (chain * 2).view(torch.int32)))
    assert nonzero > n - 100
    assert dev.progress()["launches"] >= 380
    dev.close()


def test_pipeline_more_than_64_contributions():
    _print_case("pipeline K=100")
    k, n = 100, 50_003
    rng = np.random.default_rng(32)
    x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
    xs = to_gpu_f32(x)
    out = torch.empty_like(xs[0])
    dev = fa.DeviceFairring(0, slice_size_in_bytes=64 * 1024, max_memory_allocated_in_bytes=MiB)
    dev.allreduce(out, xs, scale_mode=fa.SCALE_DIV, scale=float(k)).wait()
    assert_bits_equal(out.cpu().numpy(), oracle.sum_f32(list(x), oracle.SCALE_DIV, float(k)))
    dev.close()


@pytest.fixture(params=[None, 1 << 20, 40960], ids=["scratch-default", "scratch-1MiB", "scratch-40KiB"])
def chain_scratch(request, monkeypatch):
    # the scratch buffer that carries a chain's partial result (8 MiB per stream by default);
    # small ones make the tensors of these tests span several pieces of it
    if request.param is None:
        monkeypatch.delenv("FAIRRING_CHAIN_SCRATCH_BYTES", raising=False)
    else:
        monkeypatch.setenv("FAIRRING_CHAIN_SCRATCH_BYTES", str(request.param))
    return request.param


@pytest.mark.parametrize("alias", [3, 64, 69])
@pytest.mark.parametrize("shift", [0, 3])
def test_pipeline_in_place_with_more_than_64_contributions(alias, shift, chain_scratch):
    # reduced in place into contribution `alias`; from index 64 on, that contribution is only
    # read by the second launch of the chain, so the partial result of the first must not
    # land in it (it travels through a scratch buffer, a piece at a time)
    _print_case("pipeline in place, K=70", alias, shift, chain_scratch)
    k, n = 70, 700_001
    rng = np.random.default_rng(33 + alias)
    x = (rng.standard_normal((k, n + shift)) * 0.01).astype(np.float32)
    xs = [t[shift:] for t in to_gpu_f32(x)]
    dev = fa.DeviceFairring(0, slice_size_in_bytes=2 * MiB, max_memory_allocated_in_bytes=4 * MiB)
    dev.allreduce(xs[alias], xs, scale_mode=fa.SCALE_DIV, scale=float(k)).wait()
    assert_bits_equal(xs[alias].cpu().numpy(),
                      oracle.sum_f32(list(x[:, shift:]), oracle.SCALE_DIV, float(k), threads=8))
    for i in (0, 65):
        if i != alias:   # the other contributions are untouched
            assert_bits_equal(xs[i].cpu().numpy(), x[i, shift:])
    dev.close()


@pytest.mark.parametrize("kind,tdt", [("bf16", torch.bfloat16), ("f16", torch.float16)])
@pytest.mark.parametrize("shift", [0, 5])
def test_pipeline_half_types_round_once_over_a_chain(kind, tdt, shift, chain_scratch):
    # more contributions than one launch takes: the partial sums travel in fp32 between the
    # launches, so the result is the single fp32 fold with one rounding (at::sum_out over
    # [K, n]), not a fold that rounds to the storage type after every 64 terms
    _print_case("half-type chain", kind, shift)
    k, n = 150, 600_011
    rng = np.random.default_rng(34 + shift)
    x = (rng.standard_normal((k, n + shift)) * 0.01).astype(np.float32)
    bits = oracle.np_f32_to_bf16_rne(x).reshape(x.shape) if kind == "bf16" else \
        x.astype(np.float16).view(np.uint16)
    xs = [_np_to_gpu(r, tdt)[shift:] for r in bits]
    host = list(bits[:, shift:])
    out = torch.empty(n + shift, dtype=tdt, device=DEV)[shift:]
    dev = fa.DeviceFairring(0, slice_size_in_bytes=MiB, max_memory_allocated_in_bytes=2 * MiB)
    for mode, omode, s in ((fa.SCALE_NONE, oracle.SCALE_NONE, 1.0),
                           (fa.SCALE_DIV, oracle.SCALE_DIV, float(k)),
                           (fa.SCALE_PRE_MUL, oracle.SCALE_PRE_MUL, 1.0 / 128)):
        dev.allreduce(out, xs, scale_mode=mode, scale=s).wait()
        assert_bits_equal(_gpu_to_np(out), oracle.reduce(kind, host, "sum", omode, s),
                          "%s mode %d" % (kind, mode), half=kind == "f16")
    # in place into a late contribution, and MAX (exact in the storage type)
    dev.allreduce(out, xs, op=fa.MAX).wait()
    assert_bits_equal(_gpu_to_np(out), oracle.reduce(kind, host, "max"), kind + " max",
                      half=kind == "f16")
    want = oracle.reduce(kind, host, "sum")
    dev.allreduce(xs[140], xs).wait()
    assert_bits_equal(_gpu_to_np(xs[140]), want, kind + " in place", half=kind == "f16")
    dev.close()


@pytest.mark.parametrize("kind,tdt", [("bf16", torch.bfloat16), ("f16", torch.float16)])
@pytest.mark.parametrize("slots,carry", [(1, False), (2, True), (4, False), (6, True)])
def test_pipeline_host_staged_half_types_round_once(kind, tdt, slots, carry, chain_scratch):
    # few slots: the pinned contributions are folded batch after batch; the partial sums stay
    # in fp32 between the batches
    _print_case("half-type host staged", kind, slots, carry)
    k, n = 11, 700_001
    rng = np.random.default_rng(35 + slots)
    x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
    bits = oracle.np_f32_to_bf16_rne(x).reshape(x.shape) if kind == "bf16" else \
        x.astype(np.float16).view(np.uint16)
    hs = [torch.from_numpy(np.ascontiguousarray(r).view(np.int16)).view(tdt).pin_memory()
          for r in bits]
    slice_bytes = 512 * 1024
    dev = fa.DeviceFairring(0, slice_size_in_bytes=slice_bytes,
                            max_memory_allocated_in_bytes=slots * slice_bytes)
    assert dev.layout["staging_slots"] == slots
    want = oracle.reduce(kind, list(bits), "sum", oracle.SCALE_DIV, float(k))
    if carry:
        out = _np_to_gpu(bits[0], tdt)
        dev.allreduce_host(out, hs[1:], scale_mode=fa.SCALE_DIV, scale=float(k), carry=True).wait()
    else:
        out = torch.empty(n, dtype=tdt, device=DEV)
        dev.allreduce_host(out, hs, scale_mode=fa.SCALE_DIV, scale=float(k)).wait()
    assert_bits_equal(_gpu_to_np(out), want, kind, half=kind == "f16")
    dev.close()


@pytest.mark.parametrize("producer", ["side", "default"])
@pytest.mark.parametrize("n", [4_000_000, 50_000])
def test_pipeline_waits_for_producer_stream(producer, n):
    # The contributions are written late by the producer stream (a few milliseconds of other work
    # first); the operation is handed over at once and must see them. 4 M elements go through the
    # reduce streams (the producer's event), 50 K are launched on the producer stream itself. One
    # call of each kind beforehand: a first call takes longer than the producer is busy.
    _print_case("pipeline producer stream", producer, n)
    dev = fa.DeviceFairring(0, slice_size_in_bytes=MiB, max_memory_allocated_in_bytes=4 * MiB)
    stream = torch.cuda.Stream() if producer == "side" else torch.cuda.default_stream()
    a = torch.zeros(n, device=DEV)
    b = torch.zeros(n, device=DEV)
    out = torch.empty(n, device=DEV)
    ballast = torch.zeros(64 * MiB, device=DEV)
    try:
        with torch.cuda.stream(stream):
            ballast.add_(1.0)
            a.add_(0.0)
            dev.allreduce(out, [a, b]).wait()
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            for _ in range(30):
                ballast.add_(1.0)
            a.add_(1.0)
            b.add_(2.0)
            w = dev.allreduce(out, [a, b])
        w.wait()
        assert bool((out == 3.0).all())
    finally:
        dev.close()


@pytest.mark.parametrize("k,slots", [(1, 2), (2, 2), (5, 1), (9, 2), (9, 3), (12, 8), (64, 2)])
def test_pipeline_host_staged(k, slots):
    _print_case("pipeline host staged", k, slots)
    n = 100_003
    slot = 160_000  # bytes: the tensor needs 3 staged slices per contribution
    rng = np.random.default_rng(40 + k)
    x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
    hs = [torch.from_numpy(np.ascontiguousarray(r)).pin_memory() for r in x]
    out = torch.empty(n, dtype=torch.float32, device=DEV)
    dev = fa.DeviceFairring(0, slice_size_in_bytes=slot, max_memory_allocated_in_bytes=slot * slots)
    dev.allreduce_host(out, hs, scale_mode=fa.SCALE_DIV, scale=float(k)).wait()
    assert_bits_equal(out.cpu().numpy(), oracle.sum_f32(list(x), oracle.SCALE_DIV, float(k)))
    # second operation reuses the slots: the slot-free events must hold
    dev.allreduce_host(out, hs[::-1]).wait()
    assert_bits_equal(out.cpu().numpy(), oracle.sum_f32(list(x[::-1])))
    dev.close()


def test_pipeline_host_staged_bf16_default_layout():
    _print_case("pipeline host staged bf16")
    k, n = 8, 2_000_003
    rng = np.random.default_rng(50)
    bits = oracle.np_f32_to_bf16_rne((rng.standard_normal((k, n)) * 0.01).astype(np.float32))
    hs = [torch.from_numpy(np.ascontiguousarray(r).view(np.int16)).view(torch.bfloat16).pin_memory()
          for r in bits]
    out = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    dev = fa.DeviceFairring(0)  # 50 MiB, parallelism 16 -> 16 slots of 3,276,784 B
    assert dev.layout == dict(slot=3276784, slice=3276784, padding_slots=16, staging_slots=16)
    dev.allreduce_host(out, hs, scale_mode=fa.SCALE_MUL, scale=0.125).wait()
    assert_bits_equal(bf16_bits(out), oracle.sum_bf16(list(bits), oracle.SCALE_MUL, 0.125))
    dev.close()


def test_wait_with_a_time_limit_gives_up_with_a_report_and_can_be_repeated():
    _print_case("wait time limit")
    k, n = 4, 1_000_003
    xs = [torch.full((n,), float(i + 1), device=DEV) for i in range(k)]
    out = torch.empty(n, device=DEV)
    dev = fa.DeviceFairring(0)
    a = torch.randn(8192, 8192, device=DEV)
    torch.cuda.synchronize()
    before = dev.progress()
    try:
        fa.set_wait_timeout(0.02)
        for _ in range(60):          # keeps the producer's stream busy for a few hundred ms
            a = torch.mm(a, a).clamp_(-1, 1)
        w = dev.allreduce(out, xs)
        with pytest.raises(fa.FairringError, match="gave up after") as info:
            w.wait()
        assert info.value.code == 5   # FRG_ERR_NOT_READY
        assert "submitted" in str(info.value)
    finally:
        fa.set_wait_timeout(60)
    w.wait()
    assert float(out.min()) == 10.0 and float(out.max()) == 10.0
    after = dev.progress()
    assert after["submitted"] == before["submitted"] + 1
    assert after["enqueued"] == after["submitted"] and after["launches"] > before["launches"]
    dev.close()


def test_pipeline_many_small_operations_in_order():
    _print_case("pipeline many ops")
    dev = fa.DeviceFairring(0, slice_size_in_bytes=64 * 1024, max_memory_allocated_in_bytes=256 * 1024)
    rng = np.random.default_rng(60)
    works, wants, outs = [], [], []
    for i in range(40):
        n = int(rng.integers(1, 60000))
        k = int(rng.integers(1, 10))
        x = (rng.standard_normal((k, n))).astype(np.float32)
        xs = to_gpu_f32(x)
        out = torch.empty(n, device=DEV)
        works.append(dev.allreduce(out, xs))
        outs.append(out)
        wants.append(oracle.sum_f32(list(x)))
    for w, o, want in zip(works, outs, wants):
        w.wait()
        assert_bits_equal(o.cpu().numpy(), want)
    dev.synchronize()
    dev.close()


@pytest.mark.parametrize("n", [6_553_600 + 3, 14_000_003, 20_000_003])
def test_operations_sharing_a_tensor_keep_their_order_across_streams(n):
    # Bucket-sized operations (25 MiB: a few launches on one reduce stream, the next operation on
    # the other) and larger ones (53 and 76 MiB: launches dealt over both streams) that share a
    # tensor must run in submission order: six in-place reductions of one tensor, each with a scale
    # of its own so that the order shows in the bits; then the output of one operation as a
    # contribution of the next, and an operation that overwrites a contribution of the one before.
    # The calls are marshalled beforehand and issued back to back (a few microseconds apart, a
    # fraction of what one of them runs), and none is waited for until the end: whatever is not
    # ordered overlaps.
    _print_case("order between operations", n)
    k = 4
    g = torch.Generator(device=DEV)
    g.manual_seed(61)
    xs = [torch.empty(n, device=DEV).normal_(0, 0.01, generator=g) for _ in range(k)]
    own = xs[0].clone()
    dev = fa.DeviceFairring(0)
    try:
        scales = [0.5, 0.25, 2.0, 1.0, 4.0, 0.125]
        calls = [dev.prepare(own, [own] + xs[1:], scale_mode=fa.SCALE_MUL, scale=s) for s in scales]
        warm = torch.zeros(n, device=DEV)
        dev.allreduce(warm, [warm, warm]).wait()      # the first launch loads the code object
        torch.cuda.synchronize()
        works = [call() for call in calls]
        works[-1].wait()            # covers the earlier ones: they share its tensor
        want = xs[0].clone()
        for s_ in scales:
            for x in xs[1:]:
                want.add_(x)
            want.mul_(s_)
        assert bool(torch.equal(own.view(torch.int32), want.view(torch.int32)))
        lo, hi = n - 70_001, n
        acc = xs[0][lo:hi].cpu().numpy()
        host = [x[lo:hi].cpu().numpy() for x in xs[1:]]
        for s_ in scales:
            acc = oracle.sum_f32([acc] + host, oracle.SCALE_MUL, s_)
        assert_bits_equal(own[lo:hi].cpu().numpy(), acc)
        # read after write, then write after read
        mid = torch.zeros(n, device=DEV)
        out = torch.zeros(n, device=DEV)
        spare = xs[3].clone()
        calls = [dev.prepare(mid, xs),                        # mid = x0 + x1 + x2 + x3
                 dev.prepare(out, [mid, spare]),              # reads mid
                 dev.prepare(spare, [xs[1], xs[2]])]          # overwrites what the second reads
        torch.cuda.synchronize()
        works = [call() for call in calls]
        for w in works:
            w.wait()
        want_mid = xs[0] + xs[1]
        want_mid.add_(xs[2]).add_(xs[3])
        assert bool(torch.equal(mid.view(torch.int32), want_mid.view(torch.int32)))
        assert bool(torch.equal(out.view(torch.int32), (want_mid + xs[3]).view(torch.int32)))
        assert bool(torch.equal(spare.view(torch.int32), (xs[1] + xs[2]).view(torch.int32)))
    finally:
        dev.close()


def test_pipeline_empty_tensor_and_layout_errors():
    _print_case("pipeline empty / layout errors")
    dev = fa.DeviceFairring(0)
    e = torch.zeros(0, device=DEV)
    assert dev.allreduce(e, [e, e]).wait() is True
    dev.close()
    with pytest.raises(fa.FairringError):
        fa.DeviceFairring(0, max_padding_allocated_in_bytes=64)   # 8 padding slots < 16
    with pytest.raises(fa.FairringError):
        fa.DeviceFairring(0, slice_size_in_bytes=25 * MiB, max_memory_allocated_in_bytes=MiB)


def test_full_slice_parity_k8_25mib():
    # one real 25 MiB slice, K = 8, fused /8: the headline shape
    _print_case("full slice K=8 25MiB")
    k, n = 8, 6_553_600
    g = torch.Generator(device=DEV)
    g.manual_seed(1234)
    xs = [torch.empty(n, device=DEV).normal_(0, 0.01, generator=g) for _ in range(k)]
    out = torch.empty(n, device=DEV)
    fa.reduce_slice(out, xs, scale_mode=fa.SCALE_MUL, scale=0.125)
    torch.cuda.synchronize()
    host = [t.cpu().numpy() for t in xs]
    assert_bits_equal(out.cpu().numpy(), oracle.sum_f32(host, oracle.SCALE_MUL, 0.125, threads=8))


# ---- the other element types (fairring/utils.h:221-245) ---------------------------

def _np_to_gpu(a, tdt):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if tdt in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).to(DEV).view(tdt)
    return t.to(DEV)


def _gpu_to_np(t):
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


OTHER_TYPES = [("f16", torch.float16), ("f64", torch.float64), ("i32", torch.int32),
               ("i64", torch.int64), ("u8", torch.uint8), ("i8", torch.int8)]


def _random_of(kind, rng, k, n):
    if kind == "f16":
        x = (rng.standard_normal((k, n)) * np.exp(rng.uniform(-8, 6, (k, n)))).astype(np.float32)
        x[:, 0] = np.inf
        x[k - 1, 0] = -np.inf
        x[:, 1] = 60000.0          # overflows fp16 only after the fp32 sum is rounded
        x[0, 2] = np.nan
        return x.astype(np.float16).view(np.uint16)
    if kind == "f64":
        x = rng.standard_normal((k, n)) * np.exp(rng.uniform(-40, 40, (k, n)))
        x[0, 0] = np.nan
        return x
    info = np.iinfo(oracle.TYPES[kind][0])
    return rng.integers(info.min, int(info.max) + 1, (k, n), dtype=oracle.TYPES[kind][0])


@pytest.mark.parametrize("kind,tdt", OTHER_TYPES)
@pytest.mark.parametrize("k,n", [(1, 5), (2, 1000), (8, 70001), (13, 4099), (64, 2050)])
def test_kernel_other_types_vs_oracle(kind, tdt, k, n):
    _print_case("type", kind, k, n)
    rng = np.random.default_rng(zlib.crc32(("%s %d %d" % (kind, k, n)).encode()))
    x = _random_of(kind, rng, k, n)
    xs = [_np_to_gpu(r, tdt) for r in x]
    out = torch.empty_like(xs[0])
    half = kind == "f16"
    fa.reduce_slice(out, xs)
    torch.cuda.synchronize()
    assert_bits_equal(_gpu_to_np(out), oracle.reduce(kind, list(x)), kind + " sum", half=half)
    fa.reduce_slice(out, xs, op=fa.MAX)
    torch.cuda.synchronize()
    got, want = _gpu_to_np(out), oracle.reduce(kind, list(x), "max")
    if kind in ("f16", "f64"):   # the sign of a zero maximum is not specified
        z = (want == 0) if kind == "f64" else ((want & 0x7FFF) == 0)
        got, want = got[~z], want[~z]
    assert_bits_equal(got, want, kind + " max", half=half)
    if oracle.TYPES[kind][1]:
        fa.reduce_slice(out, xs, scale_mode=fa.SCALE_DIV, scale=float(k))
        torch.cuda.synchronize()
        assert_bits_equal(_gpu_to_np(out), oracle.reduce(kind, list(x), "sum", oracle.SCALE_DIV, float(k)),
                          kind + " div", half=half)
    else:
        with pytest.raises(fa.FairringError):
            fa.reduce_slice(out, xs, scale_mode=fa.SCALE_MUL, scale=0.5)


@pytest.mark.parametrize("kind,tdt", OTHER_TYPES)
def test_pipeline_other_types_unaligned(kind, tdt):
    _print_case("type pipeline", kind)
    k, n, shift = 5, 300_011, 3
    rng = np.random.default_rng(99)
    x = _random_of(kind, rng, k, n + shift)
    big = [_np_to_gpu(r, tdt) for r in x]
    out = torch.zeros(n + shift, dtype=tdt, device=DEV)
    dev = fa.DeviceFairring(0, slice_size_in_bytes=256 * 1024, max_memory_allocated_in_bytes=MiB)
    dev.allreduce(out[shift:], [b[shift:] for b in big]).wait()
    assert_bits_equal(_gpu_to_np(out[shift:]), oracle.reduce(kind, list(x[:, shift:])), kind,
                      half=kind == "f16")
    assert int(torch.count_nonzero(out[:shift].view(torch.uint8) if tdt != torch.uint8 else out[:shift])) == 0
    dev.close()


def test_pipeline_submitters_on_several_threads():
    # the reference is called from whichever thread autograd runs a bucket's hook on
    # (fairring/process_group.cc:131-155 takes no lock of the caller's): four threads share one
    # context, each producing its inputs on a stream of its own and submitting 40 operations of
    # mixed sizes, types and contribution counts; every result against torch's own chain on the
    # GPU (fp32, int32) or the single-rounding rule (bf16)
    import threading
    _print_case("pipeline submitters on several threads")
    dev = fa.DeviceFairring(0, slice_size_in_bytes=256 * 1024, max_memory_allocated_in_bytes=MiB,
                            num_reduce_streams=2)
    failures = []

    def worker(tid):
        try:
            torch.cuda.set_device(0)
            gen = torch.Generator(device=DEV)
            gen.manual_seed(500 + tid)
            side = torch.cuda.Stream()
            rng = np.random.default_rng(600 + tid)
            pending = []
            with torch.cuda.stream(side):
                for i in range(40):
                    k = int(rng.integers(1, 12))
                    n = int(rng.integers(1, 400_000))
                    kind = ("f32", "bf16", "i32")[int(rng.integers(0, 3))]
                    if kind == "i32":
                        xs = [torch.randint(-1000, 1000, (n,), dtype=torch.int32, device=DEV,
                                            generator=gen) for _ in range(k)]
                        want = xs[0].clone()
                        for x in xs[1:]:
                            want += x
                    else:
                        xs = [torch.randn(n, device=DEV, generator=gen) * 0.01 for _ in range(k)]
                        if kind == "bf16":
                            xs = [x.to(torch.bfloat16) for x in xs]
                        want = xs[0].float()
                        for x in xs[1:]:
                            want = want + x.float()
                        want = want.to(xs[0].dtype)
                    out = torch.empty_like(xs[0])
                    w = dev.allreduce(out, xs)          # ordered after this thread's side stream
                    pending.append((i, kind, k, n, w, out, want, xs))
                for i, kind, k, n, w, out, want, xs in pending:
                    w.wait()
                    side.synchronize()
                    view = torch.int16 if kind == "bf16" else torch.int32
                    if not bool(torch.equal(out.view(view), want.view(view))):
                        failures.append("thread %d op %d: %s k %d n %d" % (tid, i, kind, k, n))
        except Exception as e:  # noqa: BLE001  (reported by the main thread)
            failures.append("thread %d: %r" % (tid, e))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a submitter thread did not finish"
    assert not failures, failures[:5]
    assert dev.progress()["submitted"] >= 160
    dev.close()


def test_against_the_reference_call_itself_where_its_order_is_sequential():
    # doReduction calls at::sum_out over operand[K, n] (fairring/device.cc:125). On the GPU that
    # kernel folds the rows in order for K = 2 and 4 (it regroups them from K = 8 on, which is why
    # the contract is the at::add chain); there the library must equal the reference's own call
    # bit for bit. For bf16 the single rounding hides the regrouping on this data: equal for K = 8.
    _print_case("at::sum_out on the GPU")
    gen = torch.Generator(device=DEV)
    gen.manual_seed(2024)
    n = 3_000_017
    for k in (2, 4):
        st = torch.empty(k, n, device=DEV).normal_(0, 0.01, generator=gen)
        out = torch.empty(n, device=DEV)
        fa.reduce_slice(out, [st[i] for i in range(k)])
        ref = torch.sum(st, dim=0)
        torch.cuda.synchronize()
        assert bool(torch.equal(out.view(torch.int32), ref.view(torch.int32))), "fp32 K=%d" % k
    st = torch.empty(8, n, device=DEV).normal_(0, 0.01, generator=gen).to(torch.bfloat16)
    out = torch.empty(n, device=DEV, dtype=torch.bfloat16)
    fa.reduce_slice(out, [st[i] for i in range(8)])
    ref = torch.sum(st, dim=0)
    torch.cuda.synchronize()
    assert bool(torch.equal(out.view(torch.int16), ref.view(torch.int16))), "bf16 K=8"


@pytest.mark.parametrize("tdt", [torch.float32, torch.bfloat16, torch.float16, torch.float64,
                                 torch.int32, torch.int64, torch.uint8, torch.int8])
def test_max_against_amax_on_the_gpu(tdt):
    # the reference's MAX is at::amax_out over operand[K, n] (fairring/device.cc:127):
    # order-independent, NaN wins; only the sign of a zero maximum is left open (+0 == -0)
    _print_case("at::amax_out on the GPU", tdt)
    gen = torch.Generator(device=DEV)
    gen.manual_seed(77)
    n = 500_009
    for k in (1, 2, 5, 8, 13, 64, 70):
        if tdt.is_floating_point:
            st = (torch.randn(k, n, device=DEV, generator=gen) * 3).to(tdt)
            st[k // 2, 5::1001] = float("nan")
            st[0, 7::1003] = float("inf")
            st[k - 1, 9::1007] = -float("inf")
        else:
            info = torch.iinfo(tdt)
            st = torch.randint(info.min, info.max, (k, n), device=DEV, generator=gen,
                               dtype=torch.int64).to(tdt)
        out = torch.empty(n, device=DEV, dtype=tdt)
        dev = fa.DeviceFairring(0, slice_size_in_bytes=256 * 1024, max_memory_allocated_in_bytes=MiB)
        dev.allreduce(out, [st[i] for i in range(k)], op=fa.MAX).wait()
        dev.close()
        ref = torch.amax(st, dim=0)
        torch.cuda.synchronize()
        if tdt.is_floating_point:
            both_nan = out.isnan() & ref.isnan()
            zero = (out == 0) & (ref == 0)
            same = (out == ref) | both_nan
            assert bool(same.all()), "%s K=%d" % (tdt, k)
            bits = {2: torch.int16, 4: torch.int32, 8: torch.int64}[out.element_size()]
            strict = (out.view(bits) == ref.view(bits)) | both_nan | zero
            assert bool(strict.all()), "%s K=%d bits" % (tdt, k)
        else:
            assert bool(torch.equal(out, ref)), "%s K=%d" % (tdt, k)


# ---- where the rounds lie: launches placed on the 4 MiB multiples of the output's allocation ----

def _offset_in_allocation(t):
    """Bytes from the start of the hipMalloc allocation that holds `t` to its first element."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")     # the runtime torch has loaded already
    base, size = ctypes.c_void_p(), ctypes.c_size_t()
    rc = hip.hipMemGetAddressRange(ctypes.byref(base), ctypes.byref(size), ctypes.c_void_p(t.data_ptr()))
    assert rc == 0 and base.value is not None
    return t.data_ptr() - base.value


def _view_at_residue(buf, residue_bytes, n, elsize):
    """n elements of `buf` whose first byte lies `residue_bytes` past a 4 MiB multiple of the allocation."""
    off = _offset_in_allocation(buf)
    start = (residue_bytes - off) % (4 * MiB)
    assert start % elsize == 0
    return buf[start // elsize: start // elsize + n]


@pytest.mark.parametrize("kind", ["f32", "bf16"])
def test_large_operation_at_any_offset_within_its_allocation(kind):
    # An operation of 16 rounds or more starts its rounds where the output reaches a 4 MiB multiple
    # of its allocation: the first launch takes up to a whole round ahead of that point as pieces
    # (the kernel's lead), the last one what lies behind the last whole round. Offsets that leave
    # nothing, a few vectors, most of a round, and an odd number of elements ahead of the rounds.
    tdt = torch.float32 if kind == "f32" else torch.bfloat16
    elsize = 4 if kind == "f32" else 2
    k, n = 4, 100 * MiB // elsize + 12345
    g = torch.Generator(device=DEV)
    g.manual_seed(81)
    room = n + 8 * MiB // elsize
    bufs = [torch.empty(room, device=DEV).normal_(0, 0.01, generator=g).to(tdt) for _ in range(k)]
    outbuf = torch.zeros(room, dtype=tdt, device=DEV)
    dev = fa.DeviceFairring(0)
    try:
        for residue in (0, 2560, 1 * MiB + 4 * elsize, 2 * MiB, 3 * MiB + 2560, 4 * MiB - 16):
            _print_case("large operation", kind, "residue", residue)
            xs = [_view_at_residue(b, residue, n, elsize) for b in bufs]
            out = _view_at_residue(outbuf, residue, n, elsize)
            outbuf.zero_()
            before = dev.progress()["launches"]
            dev.allreduce(out, xs, scale_mode=fa.SCALE_MUL, scale=0.25).wait()
            plan = fa.plan_launches(k, n, elsize, xs[0].data_ptr(), _offset_in_allocation(out))
            assert dev.progress()["launches"] - before == len(plan) >= 6
            assert all(b == 4 for _, b in plan)
            chain = xs[0].to(torch.float32, copy=True)   # (.float() of an fp32 tensor is the tensor)
            for x in xs[1:]:
                chain.add_(x.float())
            chain.mul_(0.25)
            want = chain.to(tdt)
            it = torch.int32 if kind == "f32" else torch.int16
            assert bool(torch.equal(out.view(it), want.view(it))), residue
            # nothing outside the view was written
            lo = out.data_ptr() - outbuf.data_ptr()
            assert int(torch.count_nonzero(outbuf)) == int(torch.count_nonzero(out))
            assert lo % elsize == 0
            # and the oracle on the range around the end of the first launch's lead and rounds
            first = plan[0][0]
            a, b = max(0, first - 5000), min(n, first + 5000)
            if kind == "f32":
                host = [x[a:b].cpu().numpy() for x in xs]
                assert_bits_equal(out[a:b].cpu().numpy(), oracle.sum_f32(host, oracle.SCALE_MUL, 0.25))
            else:
                host = [bf16_bits(x[a:b]) for x in xs]
                assert_bits_equal(bf16_bits(out[a:b]), oracle.sum_bf16(host, oracle.SCALE_MUL, 0.25))
    finally:
        dev.close()


def test_stream_of_buckets_keeps_one_shape_and_switches_only_after_a_run_of_aligned_ones():
    # short operations are aligned to the 4 MiB multiples only when the four before them could be
    # too; one that cannot ends the run. 28 MiB buckets: 8 + 8 + 12 MiB aligned, 12.5 + 15.5 otherwise.
    _print_case("bucket stream: aligned after a run of four")
    k, n = 8, 28 * MiB // 4
    g = torch.Generator(device=DEV)
    g.manual_seed(82)
    room = n + 2 * MiB
    bufs = [torch.empty(room, device=DEV).normal_(0, 0.01, generator=g) for _ in range(k)]
    outbuf = torch.zeros(12 * room, device=DEV)
    dev = fa.DeviceFairring(0)
    try:
        residues = [0] * 7 + [2 * MiB] + [0] * 6       # the eighth bucket starts 2 MiB off
        launches = []
        outs, xss = [], []
        for i, residue in enumerate(residues):
            xs = [_view_at_residue(b, residue, n, 4) for b in bufs]
            out = _view_at_residue(outbuf[(i % 12) * room:], residue, n, 4)
            before = dev.progress()["launches"]
            w = dev.allreduce(out, xs, scale_mode=fa.SCALE_MUL, scale=0.125)
            w.wait()
            launches.append(dev.progress()["launches"] - before)
            chain = xs[0].clone()
            for x in xs[1:]:
                chain.add_(x)
            chain.mul_(0.125)
            assert bool(torch.equal(out.view(torch.int32), chain.view(torch.int32))), i
        assert launches == [2, 2, 2, 2, 3, 3, 3, 2, 2, 2, 2, 2, 3, 3], launches
    finally:
        dev.close()


@pytest.mark.parametrize("seed", range(6))
def test_random_sequences_of_dependent_operations_match_sequential_execution(seed):
    # Operations over ranges of a few shared buffers, issued back to back without a wait: every
    # read-after-write, write-after-read and write-after-write between them must resolve as if they
    # ran one after the other, whichever reduce streams they land on. Ranges are 8 to 40 MiB and
    # the calls are marshalled beforehand, so that an operation runs for several times the gap to
    # the next call and neighbouring operations do overlap when nothing orders them.
    _print_case("random dependent operations", seed)
    rng = np.random.default_rng(9100 + seed)
    nbuf, size = 5, 16 * MiB                              # five buffers of 64 MiB
    g = torch.Generator(device=DEV)
    g.manual_seed(9100 + seed)
    bufs = [torch.empty(size, device=DEV).normal_(0, 1.0, generator=g) for _ in range(nbuf)]
    shadow = [b.clone() for b in bufs]                    # the sequential execution, by torch
    streams = int(rng.choice([2, 3]))
    dev = fa.DeviceFairring(0, num_reduce_streams=streams)
    try:
        dev.allreduce(shadow[0][:MiB], [shadow[0][:MiB], shadow[1][:MiB]],
                      scale_mode=fa.SCALE_MUL, scale=1.0).wait()     # loads the code object
        shadow[0][:MiB] = bufs[0][:MiB] + bufs[1][:MiB]
        shadow[0][:MiB] = bufs[0][:MiB]
        calls, plan = [], []
        for _ in range(50):
            n = int(rng.integers(2 * MiB, 10 * MiB))
            ob = int(rng.integers(nbuf))
            olo = int(rng.integers(0, size - n)) // 4 * 4
            k = int(rng.integers(2, 6))
            terms = []
            for _ in range(k):
                if rng.random() < 0.25:
                    terms.append((ob, olo))               # in place: the output's own range
                    continue
                while True:
                    cb = int(rng.integers(nbuf))
                    clo = int(rng.integers(0, size - n)) // 4 * 4
                    if cb != ob or clo + n <= olo or olo + n <= clo:   # no partial overlap with `out`
                        break
                terms.append((cb, clo))
            scale = float(rng.choice([0.5, 0.25, 1.0, 2.0]))
            calls.append(dev.prepare(bufs[ob][olo:olo + n], [bufs[b][lo:lo + n] for b, lo in terms],
                                     scale_mode=fa.SCALE_MUL, scale=scale))
            plan.append((n, ob, olo, terms, scale))
        torch.cuda.synchronize()
        works = [call() for call in calls]
        for n, ob, olo, terms, scale in plan:
            acc = shadow[terms[0][0]][terms[0][1]:terms[0][1] + n].clone()
            for b, lo in terms[1:]:
                acc.add_(shadow[b][lo:lo + n])
            acc.mul_(scale)
            shadow[ob][olo:olo + n] = acc
        for w in works:
            w.wait()
        for i in range(nbuf):
            assert bool(torch.equal(bufs[i].view(torch.int32), shadow[i].view(torch.int32))), i
    finally:
        dev.close()


class HeldCommandThread:
    """Keeps the pipeline's command thread inside the completion callback of an operation
    (24 MiB moved: it goes through the command thread, not the caller's stream) until
    release() is called, so that whatever is submitted meanwhile is waiting in the queue when
    the thread takes up work again: what the command thread finds there does not depend on
    how fast this thread is today."""

    def __init__(self, dev):
        import threading
        self.entered, self.gate = threading.Event(), threading.Event()
        self.buf = torch.zeros(2 * MiB, device=DEV)

        def held(user, status, stream):
            self.entered.set()
            self.gate.wait(60)

        self.work = dev.allreduce(self.buf, [self.buf, self.buf], done=held)
        assert self.entered.wait(60), "the completion callback never ran"

    def release(self):
        self.gate.set()
        self.work.wait()


def _hold(stream, ballast, times=30):
    """Keeps `stream` busy for a few milliseconds (elementwise passes over 256 MiB)."""
    with torch.cuda.stream(stream):
        for _ in range(times):
            ballast.add_(1.0)


def test_small_operation_with_nothing_in_flight_runs_on_the_callers_stream():
    # One launch that moves at most 16 MiB, with the pipeline idle, is launched by the call itself
    # on the producer stream (no reduce stream, no event between streams). Whatever comes next
    # from another stream is still ordered after it, and synchronize() covers it.
    _print_case("small operation on the caller's stream")
    g = torch.Generator(device=DEV)
    g.manual_seed(77)
    small, big, k = 100_003, 8_000_000, 4
    xs = [torch.empty(big, device=DEV).normal_(0, 0.01, generator=g) for _ in range(k)]
    ballast = [torch.zeros(64 * MiB, device=DEV) for _ in range(2)]
    p, q = torch.cuda.Stream(), torch.cuda.Stream()
    dev = fa.DeviceFairring(0)
    torch.cuda.synchronize()
    try:
        # read after write across streams: the small result feeds a large operation
        mid = torch.zeros(big, device=DEV)
        out = torch.zeros(big, device=DEV)
        # Every kind of call once beforehand: a first call takes milliseconds (code objects are
        # loaded), longer than the producer is held up below, and would hide a missing order.
        for s_ in (p, q):
            dev.allreduce(mid[:small], [x[:small] for x in xs], stream=s_).wait()
            dev.allreduce(out, [mid, xs[1]], stream=s_).wait()
            _hold(s_, ballast[0], times=2)
        dev.synchronize()
        mid.zero_()
        out.zero_()
        torch.cuda.synchronize()
        _hold(p, ballast[0])
        before = dev.progress()
        w0 = dev.allreduce(mid[:small], [x[:small] for x in xs], scale_mode=fa.SCALE_MUL,
                           scale=0.25, stream=p)
        after = dev.progress()
        assert after["on_callers_stream"] == before["on_callers_stream"] + 1
        assert after["submitted"] == after["enqueued"] == before["submitted"] + 1
        assert w0.is_completed()                       # enqueued, on p, behind the ballast
        w1 = dev.allreduce(out, [mid, xs[1]], stream=q)   # 96 MB: through the pipeline
        assert dev.progress()["on_callers_stream"] == after["on_callers_stream"]
        w1.wait()
        want_mid = xs[0][:small] + xs[1][:small]
        want_mid.add_(xs[2][:small]).add_(xs[3][:small]).mul_(0.25)
        assert bool(torch.equal(out[:small].view(torch.int32),
                                (want_mid + xs[1][:small]).view(torch.int32)))
        assert bool(torch.equal(out[small:].view(torch.int32), xs[1][small:].view(torch.int32)))
        host = [x[:small].cpu().numpy() for x in xs]
        assert_bits_equal(mid[:small].cpu().numpy(), oracle.sum_f32(host, oracle.SCALE_MUL, 0.25))
        dev.synchronize()
        torch.cuda.synchronize()

        # two small in-place operations on one tensor from two streams, the first held up
        own = xs[0][:small].clone()
        torch.cuda.synchronize()
        _hold(p, ballast[0])
        before = dev.progress()["on_callers_stream"]
        dev.allreduce(own, [own] + [x[:small] for x in xs[1:]], scale_mode=fa.SCALE_MUL, scale=0.5,
                      stream=p)
        w = dev.allreduce(own, [own] + [x[:small] for x in xs[1:]], scale_mode=fa.SCALE_MUL,
                          scale=2.0, stream=q)
        assert dev.progress()["on_callers_stream"] == before + 2
        w.wait()                                       # q, which waited for p's operation
        acc = host[0]
        for s in (0.5, 2.0):
            acc = oracle.sum_f32([acc] + host[1:], oracle.SCALE_MUL, s)
        assert_bits_equal(own.cpu().numpy(), acc)

        # synchronize() covers what went to a caller's stream
        res = torch.zeros(small, device=DEV)
        torch.cuda.synchronize()
        _hold(q, ballast[1])
        dev.allreduce(res, [x[:small] for x in xs], stream=q)
        dev.synchronize()
        assert_bits_equal(res.cpu().numpy(), oracle.sum_f32(host))
        torch.cuda.synchronize()
    finally:
        dev.close()


@pytest.mark.parametrize("seed", range(4))
def test_random_mix_of_small_and_large_operations_from_two_streams(seed, monkeypatch):
    # Small operations (launched on the caller's stream when nothing is in flight) and large ones
    # (through the reduce streams) from two producer streams over ranges of four 4 MiB buffers, so
    # that neighbouring operations often share memory. Each episode starts from an idle pipeline
    # with a small operation behind a held-up producer (it sits on that stream for milliseconds),
    # followed by up to four operations of either kind from either stream; the result is that of
    # running them one after the other. "Small" is up to 1 MiB moved here.
    _print_case("random small and large operations from two streams", seed)
    rng = np.random.default_rng(9300 + seed)
    nbuf, size = 4, MiB
    g = torch.Generator(device=DEV)
    g.manual_seed(9300 + seed)
    bufs = [torch.empty(size, device=DEV).normal_(0, 1.0, generator=g) for _ in range(nbuf)]
    shadow = [b.clone() for b in bufs]
    ballast = [torch.zeros(64 * MiB, device=DEV) for _ in range(2)]
    producers = [torch.cuda.Stream(), torch.cuda.Stream()]
    monkeypatch.setenv("FAIRRING_INLINE_BYTES", str(MiB))
    dev = fa.DeviceFairring(0)
    warm = torch.zeros(MiB, device=DEV)
    for s_ in producers:                                  # first calls take milliseconds: not in the mix
        dev.allreduce(warm[:4096], [warm[:4096], warm[4096:8192]], stream=s_).wait()
        dev.allreduce(warm, [warm, warm], stream=s_).wait()
        _hold(s_, ballast[0], times=2)
    dev.synchronize()
    torch.cuda.synchronize()
    before = dev.progress()
    submitted = 0

    def submit(small, which):
        n = int(rng.integers(256, 50_000)) if small else int(rng.integers(100_000, 500_000))
        ob = int(rng.integers(2))                          # two of the buffers take the results,
        olo = int(rng.integers(0, size - n)) // 4 * 4      # so that ranges meet often
        k = int(rng.integers(2, 5))
        terms = []
        for _ in range(k):
            if rng.random() < 0.3:
                terms.append((ob, olo))
                continue
            while True:
                cb = int(rng.integers(nbuf))
                clo = int(rng.integers(0, size - n)) // 4 * 4
                if cb != ob or clo + n <= olo or olo + n <= clo:
                    break
            terms.append((cb, clo))
        scale = float(rng.choice([0.5, 0.25, 1.0, 2.0]))
        w = dev.allreduce(bufs[ob][olo:olo + n], [bufs[b][lo:lo + n] for b, lo in terms],
                          scale_mode=fa.SCALE_MUL, scale=scale, stream=producers[which])
        acc = shadow[terms[0][0]][terms[0][1]:terms[0][1] + n].clone()
        for b, lo in terms[1:]:
            acc.add_(shadow[b][lo:lo + n])
        acc.mul_(scale)
        shadow[ob][olo:olo + n] = acc
        return w

    try:
        import time
        for episode in range(30):
            dev.synchronize()                              # the pipeline runs empty
            torch.cuda.synchronize()
            # and stays so for longer than the rule stays off after a reduce stream was found
            # busy (200 us), so that the episode's first operation is one it applies to for sure
            time.sleep(0.002)
            first = int(rng.integers(2))
            _hold(producers[first], ballast[first], times=20)
            works = [submit(True, first)]
            for _ in range(int(rng.integers(1, 5))):
                which = int(rng.integers(2))
                if rng.random() < 0.2:
                    _hold(producers[which], ballast[which], times=10)
                works.append(submit(rng.random() < 0.5, which))
            submitted += len(works)
            for w in works:
                w.wait()
        dev.synchronize()
        torch.cuda.synchronize()
        done = dev.progress()
        for i in range(nbuf):
            assert bool(torch.equal(bufs[i].view(torch.int32), shadow[i].view(torch.int32))), i
        assert done["submitted"] - before["submitted"] == submitted
        # every episode's first operation at least
        assert 30 <= done["on_callers_stream"] - before["on_callers_stream"] < submitted
    finally:
        dev.close()


@pytest.mark.parametrize("order", ["descending", "ascending", "in_place"])
def test_neighbouring_buckets_waiting_in_the_queue_run_as_one(order):
    # A gradient handed over bucket by bucket faster than the buckets run (calls marshalled
    # beforehand, issued a few microseconds apart): the command thread finds runs of buckets that
    # continue one another waiting in its queue and cuts its launches from their joint range.
    # Every bucket still completes, and the result is the one of running them separately.
    _print_case("neighbouring buckets run as one", order)
    k, bucket, count = 4, 6_553_600, 40                      # 40 buckets of 25 MiB: 1 GB per tensor
    n = bucket * count + 12_345                              # and a ragged first one
    g = torch.Generator(device=DEV)
    g.manual_seed(17)
    xs = [torch.empty(n, device=DEV).normal_(0, 0.01, generator=g) for _ in range(k)]
    want = (xs[0] + xs[1]).add_(xs[2]).add_(xs[3]).mul_(0.25)
    out = xs[0].clone() if order == "in_place" else torch.zeros(n, device=DEV)
    spans = [(n - 12_345, n)] + [(n - 12_345 - (i + 1) * bucket, n - 12_345 - i * bucket)
                                 for i in range(count)]
    if order == "ascending":
        spans.reverse()
    dev = fa.DeviceFairring(0)
    try:
        calls = [dev.prepare(out[lo:hi], ([out[lo:hi]] if order == "in_place" else [xs[0][lo:hi]])
                             + [x[lo:hi] for x in xs[1:]], scale_mode=fa.SCALE_MUL, scale=0.25)
                 for lo, hi in spans]
        warm = torch.zeros(bucket, device=DEV)
        dev.allreduce(warm, [warm, warm]).wait()
        torch.cuda.synchronize()
        before = dev.progress()
        # the command thread is held until every bucket is waiting in its queue
        held = HeldCommandThread(dev)
        works = [call() for call in calls]
        held.release()
        for w in works:
            assert w.wait() is True
        after = dev.progress()
        assert after["enqueued"] - before["enqueued"] == len(spans) + 1
        assert after["merged"] - before["merged"] == len(spans)   # runs of 16, 16 and 9
        assert bool(torch.equal(out.view(torch.int32), want.view(torch.int32)))
        lo, hi = n - 100_000, n
        assert_bits_equal(out[lo:hi].cpu().numpy(),
                          oracle.sum_f32([x[lo:hi].cpu().numpy() for x in xs], oracle.SCALE_MUL, 0.25))
    finally:
        dev.close()


def test_neighbouring_operations_that_read_each_others_output_stay_apart():
    # z[i] += z[i - gap], bucket by bucket from the top down, with the gap four and a half buckets:
    # up to four neighbours are one elementwise operation, five are not (the fifth writes what the
    # first reads). Run one after the other, every bucket adds the ORIGINAL values below it.
    _print_case("neighbouring operations with a hazard")
    q, count = 2 * MiB, 24
    gap = 9 * q // 2
    g = torch.Generator(device=DEV)
    g.manual_seed(18)
    z = torch.empty(gap + count * q, device=DEV).normal_(0, 1.0, generator=g)
    want = z.clone()
    for i in range(count):
        lo = gap + (count - 1 - i) * q
        want[lo:lo + q] = want[lo:lo + q] + want[lo - gap:lo - gap + q]
    dev = fa.DeviceFairring(0)
    try:
        calls = []
        for i in range(count):
            lo = gap + (count - 1 - i) * q
            calls.append(dev.prepare(z[lo:lo + q], [z[lo:lo + q], z[lo - gap:lo - gap + q]]))
        warm = torch.zeros(q, device=DEV)
        dev.allreduce(warm, [warm, warm]).wait()
        torch.cuda.synchronize()
        before = dev.progress()["merged"]
        held = HeldCommandThread(dev)                      # all 24 are waiting when it lets go
        works = [call() for call in calls]
        held.release()
        for w in works:
            w.wait()
        assert bool(torch.equal(z.view(torch.int32), want.view(torch.int32)))
        assert dev.progress()["merged"] - before == count  # six runs of four
    finally:
        dev.close()


@pytest.mark.parametrize("dtype,op,scaled", [(torch.bfloat16, "sum", True), (torch.float16, "sum", False),
                                             (torch.int32, "max", False), (torch.float64, "sum", True)])
def test_joined_neighbours_give_the_bits_of_separate_operations(dtype, op, scaled, monkeypatch):
    # Whatever the element type and operator: a run of buckets that is executed as one operation
    # leaves the bits that the buckets leave one by one (FAIRRING_MERGE_OPERATIONS=1).
    _print_case("joined neighbours, other types", dtype, op)
    k, bucket, count = 5, 3_000_000, 24
    n = bucket * count
    g = torch.Generator(device=DEV)
    g.manual_seed(23)
    if dtype == torch.int32:
        xs = [torch.randint(-2**30, 2**30, (n,), device=DEV, dtype=dtype, generator=g) for _ in range(k)]
    else:
        xs = [torch.empty(n, device=DEV, dtype=torch.float32).normal_(0, 1.0, generator=g).to(dtype)
              for _ in range(k)]
    kwargs = dict(op=fa.MAX if op == "max" else fa.SUM)
    if scaled:
        kwargs.update(scale_mode=fa.SCALE_MUL, scale=0.25)
    spans = [(n - (i + 1) * bucket, n - i * bucket) for i in range(count)]
    outs = []
    for limit in ("16", "1"):
        monkeypatch.setenv("FAIRRING_MERGE_OPERATIONS", limit)
        dev = fa.DeviceFairring(0)
        try:
            out = torch.zeros(n, device=DEV, dtype=dtype)
            calls = [dev.prepare(out[lo:hi], [x[lo:hi] for x in xs], **kwargs) for lo, hi in spans]
            dev.allreduce(out[:bucket], [x[:bucket] for x in xs], **kwargs).wait()
            out.zero_()
            torch.cuda.synchronize()
            before = dev.progress()["merged"]
            held = HeldCommandThread(dev)                  # until all the buckets are queued
            works = [call() for call in calls]
            held.release()
            for w in works:
                w.wait()
            joined = dev.progress()["merged"] - before
            assert joined == (count if limit == "16" else 0)   # runs of 16 and 8, or none
            outs.append(out)
        finally:
            dev.close()
    a, b = (o.view(torch.int16 if o.element_size() == 2 else (torch.int32 if o.element_size() == 4
                                                              else torch.int64)) for o in outs)
    assert bool(torch.equal(a, b))
    lo, hi = 0, 50_000
    host = [x[lo:hi].cpu() for x in xs]
    if dtype == torch.int32:
        want = torch.stack(host).amax(dim=0)
        assert bool(torch.equal(outs[0][lo:hi].cpu(), want))


KNOBS = [{}, {"FAIRRING_INLINE_BYTES": "0"}, {"FAIRRING_MERGE_OPERATIONS": "1"},
         {"FAIRRING_SPIN_US": "0"}, {"FAIRRING_CHAIN_SCRATCH_BYTES": "65536"},
         {"FAIRRING_INLINE_BYTES": "0", "FAIRRING_MERGE_OPERATIONS": "1", "FAIRRING_SPIN_US": "0"}]


@pytest.mark.parametrize("knobs", KNOBS, ids=lambda kv: ",".join("%s=%s" % (k[9:], v) for k, v in kv.items()) or "defaults")
def test_results_do_not_depend_on_the_pipelines_knobs(knobs, monkeypatch):
    # One fixed mix of operations (small ones, a gradient's buckets in place, a whole gradient
    # into a separate output, a gathered bucket; from two producer streams that are kept busy;
    # the command thread held once so that buckets queue up) under every host-side knob's other
    # setting: the knobs choose streams, launch shapes and who launches, never the bits.
    _print_case("knob independence", knobs)
    for key, value in knobs.items():
        monkeypatch.setenv(key, value)
    k = 4
    g = torch.Generator(device=DEV)
    g.manual_seed(4242)
    bucket, count = 6_553_600, 6
    grad = [torch.empty(bucket * count + 777, device=DEV).normal_(0, 0.01, generator=g) for _ in range(k)]
    whole = [torch.empty(20_000_003, device=DEV).normal_(0, 0.01, generator=g) for _ in range(k)]
    small = [torch.empty(300_000, device=DEV).normal_(0, 0.01, generator=g) for _ in range(k)]
    host = {name: [t.cpu().numpy() for t in ts] for name, ts in (("grad", grad), ("whole", whole), ("small", small))}
    ballast = torch.zeros(64 * MiB, device=DEV)
    producers = [torch.cuda.Stream(), torch.cuda.Stream()]
    small_out = torch.zeros(300_000, device=DEV)
    whole_out = torch.empty_like(whole[0])
    pieces = [whole[2][:1_000_000].clone(), whole[2][1_000_000:1_000_003].clone(),
              whole[2][1_000_003:3_000_000].clone()]
    gathered_out = torch.empty(3_000_000, device=DEV)
    torch.cuda.synchronize()      # everything above was made on the default stream
    dev = fa.DeviceFairring(0)
    try:
        works = []
        # small operations from a busy producer, in place and not
        _hold(producers[0], ballast, times=5)
        cuts = [(0, 1000), (1000, 5_096), (5_096, 70_001), (70_001, 300_000)]
        for i, (lo, hi) in enumerate(cuts):
            works.append(dev.allreduce(small_out[lo:hi], [t[lo:hi] for t in small],
                                       scale_mode=fa.SCALE_MUL, scale=0.25, stream=producers[i % 2]))
        # a gradient's buckets, in place into contribution 0, from the other busy producer,
        # queued behind a held command thread
        _hold(producers[1], ballast, times=5)
        held = HeldCommandThread(dev)
        n = grad[0].numel()
        spans = [(n - 777, n)] + [(n - 777 - (i + 1) * bucket, n - 777 - i * bucket) for i in range(count)]
        for lo, hi in spans:
            works.append(dev.allreduce(grad[0][lo:hi], [t[lo:hi] for t in grad],
                                       scale_mode=fa.SCALE_MUL, scale=0.25, stream=producers[1]))
        held.release()
        # a whole gradient into a separate output
        works.append(dev.allreduce(whole_out, whole, scale_mode=fa.SCALE_DIV, scale=4.0,
                                   stream=producers[0]))
        # a bucket whose own contribution is read from three tensors of its own
        works.append(dev.allreduce_gathered(gathered_out, [t[:3_000_000] for t in whole], 2, pieces,
                                            scale_mode=fa.SCALE_MUL, scale=0.25, stream=producers[0]))
        for w in works:
            w.wait()
        dev.synchronize()
        torch.cuda.synchronize()
        assert_bits_equal(small_out.cpu().numpy(), oracle.sum_f32(host["small"], oracle.SCALE_MUL, 0.25), "small")
        assert_bits_equal(grad[0].cpu().numpy(), oracle.sum_f32(host["grad"], oracle.SCALE_MUL, 0.25, threads=16), "buckets")
        assert_bits_equal(whole_out.cpu().numpy(), oracle.sum_f32(host["whole"], oracle.SCALE_DIV, 4.0, threads=16), "whole")
        assert_bits_equal(gathered_out.cpu().numpy(),
                          oracle.sum_f32([h[:3_000_000] for h in host["whole"]], oracle.SCALE_MUL, 0.25, threads=16),
                          "gathered")
    finally:
        dev.close()


def test_results_do_not_depend_on_the_tile_runs():
    # The blocks of one XCD take runs of 2^r consecutive tiles per round (r = 6 by default):
    # a permutation of which block reduces which tile, nothing else. Sizes around the groups
    # of 512 tiles the permutation works in, off-boundary starts, fp32 and bf16.
    _print_case("tile runs")
    from fairring_amd import _capi
    rng = np.random.default_rng(66)
    k = 8
    try:
        for n, skew in ((2 * 1024 * 1024 + 5, 0), (3 * 1024 * 1024 + 77, 3), (25 * MiB // 4, 0), (8 * MiB // 4 * 3, 1)):
            x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
            want = oracle.sum_f32(list(x), oracle.SCALE_MUL, 0.125, threads=16)
            bits = oracle.np_f32_to_bf16_rne(x)
            wantb = oracle.sum_bf16(list(bits), oracle.SCALE_MUL, 0.125, threads=16)
            for runs in (6, 0, 3, 9):
                _capi.check(_capi.lib().frg_set_tile_runs(runs))
                xs = [torch.empty(n + 8, device=DEV)[skew:skew + n].copy_(torch.from_numpy(r)) for r in x]
                out = torch.empty(n + 8, device=DEV)[skew:skew + n]
                fa.reduce_slice(out, xs, scale_mode=fa.SCALE_MUL, scale=0.125)
                torch.cuda.synchronize()
                assert_bits_equal(out.cpu().numpy(), want, "fp32 n=%d runs=%d" % (n, runs))
                xb = to_gpu_bf16(bits)
                ob = torch.empty_like(xb[0])
                fa.reduce_slice(ob, xb, scale_mode=fa.SCALE_MUL, scale=0.125)
                torch.cuda.synchronize()
                assert_bits_equal(bf16_bits(ob), wantb, "bf16 n=%d runs=%d" % (n, runs))
    finally:
        _capi.lib().frg_set_tile_runs(6)


@pytest.mark.parametrize("kind", ["f32", "bf16", "f16"])
def test_results_do_not_depend_on_the_mixed_loads(kind):
    # The form of the main loop that mixes the loads of a lane's two vectors (by default for
    # contributions that lie close together) against the plain form, forced on and off for
    # every launch: 2, 4 and 8 contributions (the variants that have it) and 3 (which has not),
    # no scale, x1/K and every term x1/K, off-boundary starts, in place into each contribution in
    # turn (all loads come before both stores), one launch and the pipeline with a bucket and a
    # long tensor.
    _print_case("mixed loads", kind)
    from fairring_amd import _capi
    tdt = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[kind]
    rng = np.random.default_rng(67)

    def values(k, n):
        x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
        if kind == "f32":
            return x
        if kind == "bf16":
            return oracle.np_f32_to_bf16_rne(x).reshape(k, n)
        return x.astype(np.float16).view(np.uint16)

    def gpu(a, skew):
        t = torch.from_numpy(np.ascontiguousarray(a))
        if kind != "f32":
            t = t.view(torch.int16).view(tdt)
        buf = torch.empty(a.size + 16, dtype=tdt, device=DEV)
        buf[skew:skew + a.size].copy_(t)
        return buf[skew:skew + a.size]

    def host(t):
        return t.cpu().numpy() if kind == "f32" else t.view(torch.int16).cpu().numpy().view(np.uint16)

    dev = fa.DeviceFairring(0, slice_size_in_bytes=25 * MiB, max_memory_allocated_in_bytes=50 * MiB)
    try:
        for k in (8, 4, 2, 3):
            for n, skew in ((3 * 1024 * 1024 + 77, 0), (25 * MiB // 4, 1), (40 * MiB + 5, 0)):
                x = values(k, n)
                for mode, omode, sc in ((fa.SCALE_NONE, oracle.SCALE_NONE, 1.0),
                                        (fa.SCALE_MUL, oracle.SCALE_MUL, 1.0 / k),
                                        (fa.SCALE_PRE_MUL, oracle.SCALE_PRE_MUL,
                                         float(np.float32(1) / np.float32(k)))):
                    want = oracle.reduce(kind, list(x), "sum", omode, sc)
                    for mixed in (1, 0, -1):
                        _capi.check(_capi.lib().frg_set_mixed_loads(mixed))
                        xs = [gpu(r, skew) for r in x]
                        out = torch.zeros(n + 16, dtype=tdt, device=DEV)[skew:skew + n]
                        fa.reduce_slice(out, xs, scale_mode=mode, scale=sc)
                        torch.cuda.synchronize()
                        what = "%s k=%d n=%d mixed=%d" % (kind, k, n, mixed)
                        assert_bits_equal(host(out), want, what, half=kind == "f16")
                        out.zero_()
                        dev.allreduce(out, xs, scale_mode=mode, scale=sc).wait()
                        assert_bits_equal(host(out), want, what + " pipeline", half=kind == "f16")
                        j = int(rng.integers(0, k))       # in place into contribution j
                        dev.allreduce(xs[j], xs, scale_mode=mode, scale=sc).wait()
                        assert_bits_equal(host(xs[j]), want, what + " in place", half=kind == "f16")
    finally:
        _capi.lib().frg_set_mixed_loads(-1)
        dev.close()

