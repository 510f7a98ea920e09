"""GPU parity of the DDP hook arithmetic folded into the reduction: the
pre-scale modes and the reduction with bf16 / fp16 compression on either side
(torch:distributed/algorithms/ddp_comm_hooks/default_hooks.py:18-93), through
the C ABI against the CPU oracle. Bit-exact.
"""
import numpy as np
import pytest
import torch

import oracle
from conftest import assert_bits_equal

pytestmark = pytest.mark.gpu

fa = pytest.importorskip("fairring_amd")

DEV = "cuda:0"
MiB = 1024 * 1024
WIRES = [("bf16", torch.bfloat16), ("f16", torch.float16)]


def _print_case(*a):
    print("[case]", *a, flush=True)


def wide_f32(rng, shape, special=True):
    x = (rng.standard_normal(shape) * np.exp(rng.uniform(-12, 12, shape))).astype(np.float32)
    if special:
        lanes = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-42], np.float32)
        flat = x.reshape(-1)
        m = min(flat.size, lanes.size)
        flat[:m] = lanes[:m]
    return x


def to_wire_bits(x, wire):
    if wire == "bf16":
        return oracle.np_f32_to_bf16_rne(x).reshape(x.shape)
    with np.errstate(over="ignore"):
        return x.astype(np.float16).view(np.uint16)


def gpu_f32(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def gpu_wire(bits, tdt):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(DEV).view(tdt)


def bits_of(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


# ---- pre-scale -------------------------------------------------------------------------------

@pytest.mark.parametrize("k", [1, 2, 3, 4, 6, 8, 17, 64])
@pytest.mark.parametrize("n", [5, 4099, 262147])
def test_pre_scale_f32(k, n):
    _print_case("pre-scale f32", k, n)
    rng = np.random.default_rng(7000 + 10 * k + n)
    x = wide_f32(rng, (k, n))
    xs = [gpu_f32(r) for r in x]
    out = torch.empty_like(xs[0])
    fa.reduce_slice(out, xs, scale_mode=fa.SCALE_PRE_DIV, scale=float(k))
    torch.cuda.synchronize()
    assert_bits_equal(out.cpu().numpy(), oracle.sum_f32(list(x), oracle.SCALE_PRE_DIV, float(k)),
                      "pre-div")
    s = float(np.float32(1) / np.float32(k))
    fa.reduce_slice(out, xs, scale_mode=fa.SCALE_PRE_MUL, scale=s)
    torch.cuda.synchronize()
    assert_bits_equal(out.cpu().numpy(), oracle.sum_f32(list(x), oracle.SCALE_PRE_MUL, s), "pre-mul")


@pytest.mark.parametrize("kind,tdt", WIRES + [("f64", torch.float64)])
@pytest.mark.parametrize("k", [2, 4, 7, 8, 33])
def test_pre_scale_other_floating_types(kind, tdt, k):
    _print_case("pre-scale", kind, k)
    n = 70001
    rng = np.random.default_rng(7100 + k)
    x = wide_f32(rng, (k, n))
    if kind == "f64":
        h = x.astype(np.float64)
        xs = [torch.from_numpy(r.copy()).to(DEV) for r in h]
    else:
        h = to_wire_bits(x, kind)
        xs = [gpu_wire(r, tdt) for r in h]
    out = torch.empty_like(xs[0])
    for mode, omode, s in ((fa.SCALE_PRE_DIV, oracle.SCALE_PRE_DIV, float(k)),
                           (fa.SCALE_PRE_MUL, oracle.SCALE_PRE_MUL,
                            float(np.float32(1) / np.float32(k)))):
        fa.reduce_slice(out, xs, scale_mode=mode, scale=s)
        torch.cuda.synchronize()
        got = out.cpu().numpy() if kind == "f64" else bits_of(out)
        assert_bits_equal(got, oracle.reduce(kind, list(h), "sum", omode, s),
                          "%s mode %d" % (kind, mode), half=kind == "f16")


def test_pre_scale_pipeline_chain_and_rejections():
    _print_case("pre-scale pipeline")
    k, n = 150, 100_003      # more contributions than one launch takes: chained with a carry
    rng = np.random.default_rng(7200)
    x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
    xs = [gpu_f32(r) for r in x]
    out = torch.empty_like(xs[0])
    dev = fa.DeviceFairring(0, slice_size_in_bytes=128 * 1024, max_memory_allocated_in_bytes=MiB)
    dev.allreduce(out, xs, scale_mode=fa.SCALE_PRE_DIV, scale=float(k)).wait()
    assert_bits_equal(out.cpu().numpy(), oracle.sum_f32(list(x), oracle.SCALE_PRE_DIV, float(k)))
    ints = [torch.ones(16, dtype=torch.int32, device=DEV)] * 2
    with pytest.raises(fa.FairringError):
        dev.allreduce(torch.empty_like(ints[0]), ints, scale_mode=fa.SCALE_PRE_MUL, scale=0.5)
    with pytest.raises(fa.FairringError):
        dev.allreduce(out, xs[:2], op=fa.MAX, scale_mode=fa.SCALE_PRE_MUL, scale=0.5)
    host = [torch.zeros(n).pin_memory() for _ in range(2)]
    with pytest.raises(fa.FairringError):
        dev.allreduce_host(out, host, scale_mode=fa.SCALE_PRE_MUL, scale=0.5)
    dev.close()


# ---- compression folded in -------------------------------------------------------------------

def _compressed_case(wire, tdt, k, n, raw, rng, shift=0, in_place=True, out_f32=True,
                     mode="div"):
    """Returns (got, want): raw contribution `raw` (or -1), everything shifted by `shift`
    elements off its allocation."""
    x = wide_f32(rng, (k, n + shift))
    peers_bits = to_wire_bits(x, wire)
    contribs_np = [peers_bits[i, shift:] for i in range(k)]
    contribs = [gpu_wire(peers_bits[i], tdt)[shift:] for i in range(k)]
    if raw >= 0:
        contribs_np[raw] = x[raw, shift:]
        contribs[raw] = gpu_f32(x[raw])[shift:]
    if mode == "div":
        fmode, omode, s = fa.SCALE_DIV, oracle.SCALE_DIV, float(k)
    elif mode == "mul":
        fmode, omode, s = fa.SCALE_MUL, oracle.SCALE_MUL, float(np.float32(1) / np.float32(k))
    else:
        fmode, omode, s = fa.SCALE_NONE, oracle.SCALE_NONE, 1.0
    if out_f32:
        out = contribs[raw] if (in_place and raw >= 0) else torch.empty(n + shift, device=DEV)[shift:]
    else:
        out = torch.empty(n + shift, dtype=tdt, device=DEV)[shift:]
    fa.reduce_slice_compressed(out, contribs, raw, scale_mode=fmode, scale=s, wire_dtype=tdt)
    torch.cuda.synchronize()
    want = oracle.compressed_sum(contribs_np, raw, wire, omode, s, out_f32=out_f32)
    got = out.cpu().numpy() if out_f32 else bits_of(out)
    return got, want


@pytest.mark.parametrize("wire,tdt", WIRES)
def test_compressed_results_do_not_depend_on_the_tile_runs(wire, tdt):
    # Whole rounds of the 512-block grid (2,048 elements per tile): the blocks of one XCD take
    # runs of consecutive tiles, a permutation of which block reduces which tile and nothing
    # else. Two and three rounds plus a ragged rest, an off-boundary start, the hook's own
    # shape (K = 8, fp32 bucket in place) and the general body (K = 5, wire output).
    _print_case("compressed, tile runs", wire)
    from fairring_amd import _capi
    rng = np.random.default_rng(8100)
    try:
        for runs in (6, 0, 3, 5):
            _capi.check(_capi.lib().frg_set_tile_runs(runs))
            for n, shift in ((2 * 512 * 2048 + 77, 0), (3 * 512 * 2048 + 4099, 8)):
                got, want = _compressed_case(wire, tdt, 8, n, 3, rng, shift=shift, mode="mul")
                assert_bits_equal(got, want, "%s K 8 n %d runs %d" % (wire, n, runs))
            got, want = _compressed_case(wire, tdt, 5, 2 * 512 * 2048 + 9, 1, rng, out_f32=False)
            assert_bits_equal(got, want, "%s K 5 wire output, runs %d" % (wire, runs))
    finally:
        _capi.lib().frg_set_tile_runs(6)


@pytest.mark.parametrize("wire,tdt", WIRES)
@pytest.mark.parametrize("k", [1, 2, 3, 4, 8, 9, 17, 64])
@pytest.mark.parametrize("n", [1, 7, 8, 9, 2051, 262147])
def test_compressed_sizes(wire, tdt, k, n):
    _print_case("compressed sizes", wire, k, n)
    rng = np.random.default_rng(8000 + 100 * k + n)
    for raw in sorted({0, k // 2, k - 1}):
        got, want = _compressed_case(wire, tdt, k, n, raw, rng)
        assert_bits_equal(got, want, "%s k %d n %d raw %d" % (wire, k, n, raw))


@pytest.mark.parametrize("wire,tdt", WIRES)
@pytest.mark.parametrize("k", [2, 4, 8])
def test_compressed_hook_shapes_with_the_own_term_at_every_rank(wire, tdt, k):
    # the shapes with compile-time variants (raw fp32 bucket + 1, 3 or 7 peers, fp32 output):
    # the own term joins the fold at its rank's place, whichever that is; a ragged length so
    # that the element-wise edges run the same variant
    _print_case("compressed hook shapes", wire, k)
    rng = np.random.default_rng(8800 + k)
    for raw in range(k):
        for mode in ("mul", "none"):         # the two scale modes those variants are compiled for
            for in_place in (True, False):
                got, want = _compressed_case(wire, tdt, k, 70003, raw, rng, in_place=in_place,
                                             mode=mode)
                assert_bits_equal(got, want, "%s k %d raw %d %s in place %s" % (
                    wire, k, raw, mode, in_place))
    got, want = _compressed_case(wire, tdt, k, 70003, k - 1, rng, shift=3, mode="mul")
    assert_bits_equal(got, want, "%s k %d off the 16-byte boundary" % (wire, k))


@pytest.mark.parametrize("wire,tdt", WIRES)
def test_compressed_output_kinds_and_modes(wire, tdt):
    _print_case("compressed outputs", wire)
    rng = np.random.default_rng(8100)
    k, n = 8, 70001
    for mode in ("div", "mul", "none"):
        got, want = _compressed_case(wire, tdt, k, n, 3, rng, in_place=False, mode=mode)
        assert_bits_equal(got, want, "separate fp32 output, " + mode)
        got, want = _compressed_case(wire, tdt, k, n, 3, rng, out_f32=False, mode=mode)
        assert_bits_equal(got, want, "wire output, " + mode, half=True)
    # no raw contribution: the plain reduction of the wire type, widened or not
    got, want = _compressed_case(wire, tdt, k, n, -1, rng, mode="none")
    assert_bits_equal(got, want, "all peers -> fp32")
    got, want = _compressed_case(wire, tdt, k, n, -1, rng, out_f32=False, mode="none")
    assert_bits_equal(got, want, "all peers -> wire", half=True)


@pytest.mark.parametrize("wire,tdt", WIRES)
@pytest.mark.parametrize("shift", [1, 2, 3, 4, 5, 7])
def test_compressed_unaligned(wire, tdt, shift):
    # every tensor shifted by the same number of elements off its allocation: the wire pointers
    # move by 2*shift bytes, the fp32 ones by 4*shift, and one common head of (8 - shift) mod 8
    # elements brings all of them to 16-byte boundaries (the vector variant still runs)
    _print_case("compressed unaligned", wire, shift)
    rng = np.random.default_rng(8200 + shift)
    got, want = _compressed_case(wire, tdt, 8, 10007, 2, rng, shift=shift)
    assert_bits_equal(got, want, "shift %d" % shift)
    got, want = _compressed_case(wire, tdt, 5, 10007, 4, rng, shift=shift, out_f32=False)
    assert_bits_equal(got, want, "shift %d wire out" % shift, half=True)


def test_compressed_mismatched_alignment_falls_back():
    _print_case("compressed mismatched alignment")
    rng = np.random.default_rng(8300)
    k, n = 5, 5003
    x = wide_f32(rng, (k, n + 8))
    bits = to_wire_bits(x, "bf16")
    contribs, contribs_np = [], []
    for i in range(k):
        sh = i % 5
        if i == 1:
            contribs.append(gpu_f32(x[i])[sh:sh + n])
            contribs_np.append(x[i, sh:sh + n])
        else:
            contribs.append(gpu_wire(bits[i], torch.bfloat16)[sh:sh + n])
            contribs_np.append(bits[i, sh:sh + n])
    out = torch.empty(n + 1, device=DEV)[1:]
    fa.reduce_slice_compressed(out, contribs, 1, scale_mode=fa.SCALE_DIV, scale=5.0)
    torch.cuda.synchronize()
    assert_bits_equal(out.cpu().numpy(),
                      oracle.compressed_sum(contribs_np, 1, "bf16", oracle.SCALE_DIV, 5.0))


@pytest.mark.parametrize("wire,tdt", WIRES)
def test_compressed_equals_torch_hook_on_gpu(wire, tdt):
    # the three passes of the hook run by torch on the GPU itself: cast + div_, fp32 fold with
    # one rounding, copy_ back (ATen on the GPU divides by a scalar as a multiply by 1/world).
    # All values are kept positive and well inside the normal range of the wire type: some of
    # ATen's GPU kernels round ties in the fp16 subnormal range away from zero where its CPU
    # kernels, the oracle and this library round to even (seen on a.div_(48): 5 lanes of 3 M).
    _print_case("compressed vs torch on gpu", wire)
    k, n = 6, 300_007
    g = torch.Generator(device=DEV)
    g.manual_seed(11)
    buckets = [torch.empty(n, device=DEV).normal_(0, 1, generator=g).abs_().add_(0.01)
               for _ in range(k)]
    comp = [b.to(tdt).div_(k) for b in buckets]
    acc = comp[0].float()
    for c in comp[1:]:
        acc = acc + c.float()
    want = buckets[2].clone()
    want.copy_(acc.to(tdt))
    contribs = list(comp)
    contribs[2] = buckets[2]
    fa.reduce_slice_compressed(buckets[2], contribs, 2, scale_mode=fa.SCALE_MUL,
                               scale=float(np.float32(1) / np.float32(k)))
    torch.cuda.synchronize()
    assert_bits_equal(buckets[2].cpu().numpy(), want.cpu().numpy())


@pytest.mark.parametrize("wire,tdt", WIRES)
@pytest.mark.parametrize("slice_bytes,streams", [(64 * 1024, 1), (256 * 1024, 2), (MiB, 3)])
def test_compressed_pipeline(wire, tdt, slice_bytes, streams):
    _print_case("compressed pipeline", wire, slice_bytes, streams)
    k, n, raw = 8, 1_000_003, 5
    rng = np.random.default_rng(8400)
    x = wide_f32(rng, (k, n), special=False)
    bits = to_wire_bits(x, wire)
    contribs = [gpu_wire(bits[i], tdt) for i in range(k)]
    contribs_np = [bits[i] for i in range(k)]
    contribs[raw] = gpu_f32(x[raw])
    contribs_np[raw] = x[raw]
    dev = fa.DeviceFairring(0, slice_size_in_bytes=slice_bytes,
                            max_memory_allocated_in_bytes=2 * slice_bytes,
                            num_reduce_streams=streams, max_launch_bytes=slice_bytes // 2)
    want = oracle.compressed_sum(contribs_np, raw, wire, oracle.SCALE_DIV, float(k), threads=8)
    w = dev.allreduce_compressed(contribs[raw], contribs, raw, scale_mode=fa.SCALE_DIV,
                                 scale=float(k))
    w.wait()
    assert_bits_equal(contribs[raw].cpu().numpy(), want)
    out = torch.empty(n, dtype=tdt, device=DEV)
    contribs[raw] = gpu_f32(x[raw])
    dev.allreduce_compressed(out, contribs, raw, scale_mode=fa.SCALE_DIV, scale=float(k)).wait()
    assert_bits_equal(bits_of(out), oracle.compressed_sum(contribs_np, raw, wire, oracle.SCALE_DIV,
                                                          float(k), out_f32=False, threads=8),
                      half=True)
    dev.close()


def test_compressed_error_paths():
    _print_case("compressed errors")
    n = 64
    raw = torch.zeros(n, device=DEV)
    peer = torch.zeros(n, dtype=torch.bfloat16, device=DEV)
    out = torch.zeros(n, device=DEV)
    with pytest.raises(fa.FairringError):    # raw_index out of range
        fa.reduce_slice_compressed(out, [raw, peer], 2)
    with pytest.raises(fa.FairringError):    # the raw contribution must be fp32
        fa.reduce_slice_compressed(out, [peer.half(), peer], 0)
    with pytest.raises(fa.FairringError):    # peers of two wire types
        fa.reduce_slice_compressed(out, [peer, peer.half()], -1)
    with pytest.raises(fa.FairringError):    # output neither fp32 nor of the wire type
        fa.reduce_slice_compressed(torch.zeros(n, dtype=torch.float16, device=DEV), [raw, peer], 0)
    with pytest.raises(fa.FairringError):    # pre-scale is not a mode of the compress step
        fa.reduce_slice_compressed(out, [raw, peer], 0, scale_mode=fa.SCALE_PRE_MUL, scale=0.5)
    with pytest.raises(fa.FairringError):    # fp32 output overlapping a peer's tensor
        both = torch.zeros(2 * n, dtype=torch.bfloat16, device=DEV)
        fa.reduce_slice_compressed(both.view(torch.float32), [raw, both[:n]], 0)
    with pytest.raises(fa.FairringError):    # 65 contributions
        fa.reduce_slice_compressed(out, [raw] + [peer] * 64, 0)
    # empty tensors are fine
    e = torch.zeros(0, device=DEV)
    fa.reduce_slice_compressed(e, [e, torch.zeros(0, dtype=torch.bfloat16, device=DEV)], 0)
    torch.cuda.synchronize()


def test_fp16_products_of_negative_zero_keep_their_sign():
    # -0 * s is -0. A mixed-precision fma with a +0 addend, which a compiler may pick for
    # "multiply, then convert to fp16", gives +0; every scaled fp16 path is held to -0.
    _print_case("fp16 negative zero")
    n = 4099
    neg0 = np.full(n, -0.0, np.float32)
    tiny = np.full(n, -1e-9, np.float32)          # underflows to -0 in fp16
    h = neg0.astype(np.float16).view(np.uint16)
    assert (h == 0x8000).all()
    xs = [gpu_wire(h, torch.float16)]
    out = torch.empty_like(xs[0])
    for mode, s in ((fa.SCALE_MUL, 0.5), (fa.SCALE_DIV, 3.0), (fa.SCALE_PRE_MUL, 0.5),
                    (fa.SCALE_PRE_DIV, 3.0)):
        out.fill_(1.0)
        fa.reduce_slice(out, xs, scale_mode=mode, scale=s)
        torch.cuda.synchronize()
        assert (bits_of(out) == 0x8000).all(), mode
    for src in (neg0, tiny):
        for mode, s in ((fa.SCALE_NONE, 1.0), (fa.SCALE_MUL, 0.5), (fa.SCALE_DIV, 3.0)):
            bucket = gpu_f32(src)
            fa.reduce_slice_compressed(bucket, [bucket], 0, scale_mode=mode, scale=s,
                                       wire_dtype=torch.float16)
            torch.cuda.synchronize()
            assert (bucket.cpu().numpy().view(np.uint32) == 0x80000000).all(), (mode, src[0])
