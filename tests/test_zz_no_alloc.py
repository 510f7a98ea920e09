"""frg_reduce_slice_static: the entry point that allocates nothing, against
frg_allreduce, whose context allocates the scratch buffer of the same chains.
Bit-exact; two calls in a row, the second one smaller."""
import numpy as np
import pytest
import torch

import oracle
from conftest import assert_bits_equal

pytestmark = pytest.mark.gpu

fa = pytest.importorskip("fairring_amd")
from fairring_amd import _capi  # noqa: E402

DEV = "cuda:0"
MiB = 1024 * 1024


def bits16(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def test_static_scratch_chain_matches_the_pipeline_on_two_calls_in_a_row():
    print("[case] no-alloc entry point, bf16 K = 100, two sizes", flush=True)
    k = 100
    g = torch.Generator(device=DEV)
    g.manual_seed(71)
    dev = fa.DeviceFairring(0)
    try:
        for n in (1_000_003, 70_001):          # the second call is the smaller one
            xs = [torch.empty(n, device=DEV).normal_(0, 0.01, generator=g).to(torch.bfloat16)
                  for _ in range(k)]
            want = torch.empty(n, dtype=torch.bfloat16, device=DEV)
            dev.allreduce(want, xs, scale_mode=fa.SCALE_DIV, scale=float(k)).wait()
            got = torch.full((n,), 7.0, dtype=torch.bfloat16, device=DEV)
            fa.reduce_slice_static(got, xs, scale_mode=fa.SCALE_DIV, scale=float(k))
            torch.cuda.synchronize()
            assert_bits_equal(bits16(got), bits16(want), "n = %d" % n)
            # and both against the oracle (one rounding at the end of the chain)
            host = [bits16(x) for x in xs]
            assert_bits_equal(bits16(got), oracle.sum_bf16(host, oracle.SCALE_DIV, float(k),
                                                           threads=8), "oracle, n = %d" % n)
    finally:
        dev.close()


def test_static_scratch_in_place_into_a_late_contribution_and_plain_cases():
    print("[case] no-alloc entry point, fp32 in place at rank 80; K <= 64; fp32 chain", flush=True)
    k, n = 100, 300_007
    g = torch.Generator(device=DEV)
    g.manual_seed(72)
    dev = fa.DeviceFairring(0)
    try:
        xs = [torch.empty(n, device=DEV).normal_(0, 1.0, generator=g) for _ in range(k)]
        want = torch.empty(n, device=DEV)
        dev.allreduce(want, xs).wait()
        target = xs[80]                        # read only by the second launch of the chain
        fa.reduce_slice_static(target, xs)
        torch.cuda.synchronize()
        assert_bits_equal(target.cpu().numpy(), want.cpu().numpy(), "in place at rank 80")
        # a chain that carries its partial result in `out` (fp32, separate output): any size
        xs[80] = torch.empty(n, device=DEV).normal_(0, 1.0, generator=g)
        dev.allreduce(want, xs, scale_mode=fa.SCALE_MUL, scale=0.01).wait()
        got = torch.empty(n, device=DEV)
        fa.reduce_slice_static(got, xs, scale_mode=fa.SCALE_MUL, scale=0.01)
        torch.cuda.synchronize()
        assert_bits_equal(got.cpu().numpy(), want.cpu().numpy(), "fp32 chain")
        # up to 64 contributions it is frg_reduce_slice
        fa.reduce_slice_static(got, xs[:8], op=fa.MAX)
        fa.reduce_slice(want, xs[:8], op=fa.MAX)
        torch.cuda.synchronize()
        assert_bits_equal(got.cpu().numpy(), want.cpu().numpy(), "K = 8 max")
    finally:
        dev.close()


def test_static_scratch_rejects_what_it_cannot_hold():
    print("[case] no-alloc entry point, limits", flush=True)
    cap = 8 * MiB // 4                         # fp32 accumulators of a 2-byte type
    n = cap + 1
    x = torch.zeros(n, dtype=torch.bfloat16, device=DEV)
    out = torch.zeros(n, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(fa.FairringError) as e:
        fa.reduce_slice_static(out, [x] * 65)
    assert e.value.code == _capi.ERR_INVALID and "at most %d elements" % cap in str(e.value)
    fa.reduce_slice_static(out[:cap], [x[:cap]] * 65)       # exactly what it holds
    fa.reduce_slice_static(out, [x] * 64)                   # one launch: no scratch, any size
    f = torch.zeros(3 * cap, device=DEV)
    fa.reduce_slice_static(torch.empty_like(f), [f] * 65)   # fp32 carries in `out`: any size
    torch.cuda.synchronize()
    with pytest.raises(fa.FairringError) as e:
        fa.reduce_slice_static(out[:16], [x[:16]] * 4097)
    assert e.value.code == _capi.ERR_INVALID and "4096" in str(e.value)


@pytest.mark.parametrize("dtype,kind", [(torch.bfloat16, "bf16"), (torch.float16, "f16")])
def test_static_scratch_chain_off_16_byte_boundaries(dtype, kind):
    # The output and the contributions 2, 6 and 10 bytes past a 16-byte boundary (the vector
    # variant with a scalar head, the fp32 accumulators in the scratch moved along with them),
    # and the output at another offset than the contributions (the scalar variant): the bits of
    # the pipeline's chain, and of the oracle's single fold with one rounding at the end.
    print("[case] no-alloc entry point, offsets of 2 / 6 / 10 bytes,", kind, flush=True)
    k, n = 70, 200_003
    g = torch.Generator(device=DEV)
    g.manual_seed(73)
    base = [torch.empty(n + 16, device=DEV).normal_(0, 0.05, generator=g).to(dtype) for _ in range(k)]
    dev = fa.DeviceFairring(0)
    try:
        for off, out_off in ((1, 1), (3, 3), (5, 5), (3, 0), (0, 5)):
            xs = [b[off:off + n] for b in base]
            want = torch.empty(n, dtype=dtype, device=DEV)
            dev.allreduce(want, xs, scale_mode=fa.SCALE_MUL, scale=1.0 / k).wait()
            room = torch.full((n + 16,), 3.0, dtype=dtype, device=DEV)
            got = room[out_off:out_off + n]
            fa.reduce_slice_static(got, xs, scale_mode=fa.SCALE_MUL, scale=1.0 / k)
            torch.cuda.synchronize()
            assert_bits_equal(bits16(got), bits16(want), "offsets %d / %d" % (off, out_off))
            assert_bits_equal(bits16(got), oracle.reduce(kind, [bits16(x) for x in xs], "sum",
                                                         oracle.SCALE_MUL, 1.0 / k),
                              "oracle, offsets %d / %d" % (off, out_off))
            # nothing outside the output was written
            assert bool((room[:out_off] == 3.0).all()) and bool((room[out_off + n:] == 3.0).all())
    finally:
        dev.close()


def test_static_scratch_max_in_place_into_a_late_contribution():
    # MAX carries its exact partial result; reduced in place into contribution 80, which only
    # the second launch of the chain reads, it must not land there before that launch has run.
    print("[case] no-alloc entry point, MAX in place at rank 80 (fp32 and int32)", flush=True)
    k, n = 100, 150_001
    g = torch.Generator(device=DEV)
    g.manual_seed(74)
    for dtype in (torch.float32, torch.int32):
        if dtype == torch.int32:
            xs = [torch.randint(-2**30, 2**30, (n,), device=DEV, dtype=dtype, generator=g)
                  for _ in range(k)]
        else:
            xs = [torch.empty(n, device=DEV).normal_(0, 1.0, generator=g) for _ in range(k)]
        want = torch.stack(xs).amax(dim=0)
        host = [x[:50_000].cpu().numpy() for x in xs]
        fa.reduce_slice_static(xs[80], xs, op=fa.MAX)
        torch.cuda.synchronize()
        assert bool(torch.equal(xs[80], want)), str(dtype)
        assert_bits_equal(xs[80][:50_000].cpu().numpy(),
                          oracle.reduce("f32" if dtype == torch.float32 else "i32", host, "max"), "oracle")


def test_static_scratch_chain_captured_into_a_graph_and_replayed():
    # What the entry point is for: a stream under capture. The context is created first (it
    # looks the array up, so the capture meets no set-up); the captured chain is replayed with
    # other inputs each time, with eager work and synchronisations in between, and every replay
    # is compared with the eager call on the same inputs.
    print("[case] no-alloc entry point under graph capture, three replays", flush=True)
    k, n = 70, 120_001
    g = torch.Generator(device=DEV)
    g.manual_seed(75)
    dev = fa.DeviceFairring(0)
    try:
        xs = [torch.empty(n, device=DEV).normal_(0, 0.05, generator=g).to(torch.bfloat16)
              for _ in range(k)]
        got = torch.zeros(n, dtype=torch.bfloat16, device=DEV)
        eager = torch.zeros(n, dtype=torch.bfloat16, device=DEV)
        fa.reduce_slice_static(eager, xs, scale_mode=fa.SCALE_MUL, scale=1.0 / k)   # warm
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fa.reduce_slice_static(got, xs, scale_mode=fa.SCALE_MUL, scale=1.0 / k)
        for replay in range(3):
            for x in xs[::7]:                  # eager work between the replays
                x.mul_(1.5 + replay)
            got.fill_(9.0)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            fa.reduce_slice_static(eager, xs, scale_mode=fa.SCALE_MUL, scale=1.0 / k)
            torch.cuda.synchronize()
            assert_bits_equal(bits16(got), bits16(eager), "replay %d" % replay)
            assert_bits_equal(bits16(got), oracle.sum_bf16([bits16(x) for x in xs], oracle.SCALE_MUL,
                                                           1.0 / k, threads=8), "oracle, replay %d" % replay)
    finally:
        dev.close()


KINDS = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16, "f64": torch.float64,
         "i32": torch.int32, "i64": torch.int64, "u8": torch.uint8}


def _to_gpu(kind, a, skew):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if kind in ("bf16", "f16"):
        t = t.view(torch.int16).view(KINDS[kind])
    buf = torch.empty(a.size + skew + 16, dtype=KINDS[kind], device=DEV)
    buf[skew:skew + a.size].copy_(t)
    return buf[skew:skew + a.size]


def _to_np(kind, t):
    return bits16(t) if kind in ("bf16", "f16") else t.cpu().numpy()


@pytest.mark.parametrize("seed", range(4))
def test_static_scratch_random_cases(seed):
    # Random element type, reduction, scale, number of contributions (1 to 200: up to four
    # launches chained through the static array), length, place of every buffer within 16
    # bytes, and in place or not (also into a contribution beyond the first launch's). Against
    # the oracle; consecutive cases share the array.
    rng = np.random.default_rng(9000 + seed)
    for case in range(10):
        kind = ["f32", "bf16", "f16", "f64", "i32", "i64", "u8"][int(rng.integers(0, 7))]
        floating = kind in ("f32", "bf16", "f16", "f64")
        op = "max" if rng.integers(0, 4) == 0 else "sum"
        k = int(rng.integers(1, 201)) if rng.integers(0, 3) else int(rng.integers(1, 9))
        n = int(rng.integers(1, 1 << int(rng.integers(1, 18))))
        scale = "none"
        if floating and op == "sum":
            scale = ["none", "mul", "div", "premul", "prediv"][int(rng.integers(0, 5))]
        modes = {"none": (fa.SCALE_NONE, oracle.SCALE_NONE, 1.0),
                 "mul": (fa.SCALE_MUL, oracle.SCALE_MUL, float(np.float32(1) / np.float32(k))),
                 "div": (fa.SCALE_DIV, oracle.SCALE_DIV, float(k)),
                 "premul": (fa.SCALE_PRE_MUL, oracle.SCALE_PRE_MUL, float(np.float32(1) / np.float32(k))),
                 "prediv": (fa.SCALE_PRE_DIV, oracle.SCALE_PRE_DIV, float(k))}
        mode, omode, sc = modes[scale]
        per16 = 16 // torch.empty(0, dtype=KINDS[kind]).element_size()
        in_place = int(rng.integers(0, k)) if rng.integers(0, 3) == 0 else -1
        print("[case] no-alloc entry point, random", seed, case, kind, op, scale, "k", k, "n", n,
              "in place", in_place, flush=True)
        if floating:
            x = (rng.standard_normal((k, n)) * np.exp(rng.uniform(-3, 3, (k, n)))).astype(np.float32)
            if kind == "bf16":
                x = oracle.np_f32_to_bf16_rne(x).reshape(k, n)
            elif kind == "f16":
                x = x.astype(np.float16).view(np.uint16)
            elif kind == "f64":
                x = x.astype(np.float64)
        else:
            info = np.iinfo(oracle.TYPES[kind][0])
            x = rng.integers(info.min, int(info.max) + 1, (k, n), dtype=oracle.TYPES[kind][0])
        xs = [_to_gpu(kind, x[j], int(rng.integers(0, per16))) for j in range(k)]
        room = None
        if in_place >= 0:
            out = xs[in_place]
        else:
            oskew = int(rng.integers(0, per16))
            room = torch.zeros(n + 32, dtype=KINDS[kind], device=DEV)
            out = room[oskew:oskew + n]
        fa.reduce_slice_static(out, xs, op=fa.MAX if op == "max" else fa.SUM, scale_mode=mode, scale=sc)
        torch.cuda.synchronize()
        want = oracle.reduce(kind, list(x), op, omode, sc)
        assert_bits_equal(_to_np(kind, out), want, "seed %d case %d" % (seed, case), half=kind == "f16")

