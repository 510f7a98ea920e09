"""Pins the CPU oracle (test infrastructure) before anything is compared to it.

Checks, none of which retypes the oracle's own formula:
  * golden vectors written by the installed ATen (tests/golden/make_golden.py)
  * live torch.add chain and torch.sum(dim=0) (K <= 17) from the installed torch
  * ATen's bf16 sum over dim 0 (fp32 accumulate, one rounding)
  * exact rational arithmetic + explicit round-to-nearest-even on tiny inputs
  * the all-ones / arange known answers of benchmark/benchmark.cc:130-186
  * closed forms for the layout and slicing (fairring/utils.h:258-327,
    fairring/device.cc:315-326)
"""
import struct
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle
from conftest import assert_bits_equal

F32_CASES = ["f32_k2", "f32_k3", "f32_k8", "f32_k17", "f32_k64"]
BF16_CASES = ["bf16_k2", "bf16_k8", "bf16_k64"]


@pytest.mark.parametrize("case", F32_CASES)
def test_f32_matches_golden(golden, case):
    x = golden[case + "_in"]
    k = x.shape[0]
    assert_bits_equal(oracle.sum_f32(list(x)), golden[case + "_sum"], case)
    assert_bits_equal(oracle.sum_f32(list(x), oracle.SCALE_MUL, 1.0 / k),
                      golden[case + "_mul"], case + " mul")
    assert_bits_equal(oracle.sum_f32(list(x), oracle.SCALE_DIV, float(k)),
                      golden[case + "_div"], case + " div")
    # the numpy restatement and the blocked multi-threaded chain agree too
    assert_bits_equal(oracle.np_sum_f32(list(x)), golden[case + "_sum"], case + " np")
    assert_bits_equal(oracle.sum_f32(list(x), oracle.SCALE_DIV, float(k), chain=True, threads=4),
                      golden[case + "_div"], case + " chain")


@pytest.mark.parametrize("case", BF16_CASES)
def test_bf16_matches_golden(golden, case):
    x = golden[case + "_in"]
    k = x.shape[0]
    assert_bits_equal(oracle.sum_bf16(list(x)), golden[case + "_sum"], case)
    assert_bits_equal(oracle.sum_bf16(list(x), oracle.SCALE_MUL, 1.0 / k),
                      golden[case + "_mul"], case + " mul")
    assert_bits_equal(oracle.sum_bf16(list(x), oracle.SCALE_DIV, float(k)),
                      golden[case + "_div"], case + " div")
    assert_bits_equal(oracle.np_sum_bf16(list(x), oracle.SCALE_MUL, 1.0 / k),
                      golden[case + "_mul"], case + " np")


@pytest.mark.parametrize("k", [2, 3, 8, 15, 16, 17, 32, 64])
def test_f32_matches_live_torch_chain(k):
    rng = np.random.default_rng(100 + k)
    x = (rng.standard_normal((k, 20011)) * 0.01).astype(np.float32)
    t = torch.from_numpy(x)
    acc = t[0].clone()
    for i in range(1, k):
        acc = torch.add(acc, t[i])
    assert_bits_equal(oracle.sum_f32(list(x)), acc.numpy(), "chain k=%d" % k)
    assert_bits_equal(oracle.sum_f32(list(x), oracle.SCALE_DIV, float(k)),
                      torch.div(acc, float(k)).numpy(), "div k=%d" % k)
    if k <= 17:
        # ATen's CPU sum over dim 0 keeps the sequential order up to K = 17 in
        # its vectorised body; the ragged tail lanes (numel % 64) go through a
        # multi-accumulator scalar loop that regroups, so they are left out.
        body = (x.shape[1] // 64) * 64
        assert_bits_equal(oracle.sum_f32(list(x))[:body],
                          torch.sum(t, dim=0).numpy()[:body], "sum_out k=%d" % k)


@pytest.mark.parametrize("k", [2, 8, 64])
def test_bf16_matches_aten_sum(k):
    rng = np.random.default_rng(200 + k)
    t = torch.from_numpy((rng.standard_normal((k, 10007)) * 0.01).astype(np.float32)).to(torch.bfloat16)
    bits = t.view(torch.int16).numpy().view(np.uint16)
    want = torch.sum(t, dim=0).view(torch.int16).numpy().view(np.uint16)
    assert_bits_equal(oracle.sum_bf16(list(bits)), want, "bf16 sum k=%d" % k)


def test_pow2_mul_equals_div_and_ddp_predivision():
    # For K = 2^p and no subnormal results, acc*(1/K) == acc/K == sum of x/K.
    rng = np.random.default_rng(7)
    x = (rng.standard_normal((8, 50000)) * 0.01).astype(np.float32)
    a = oracle.sum_f32(list(x), oracle.SCALE_MUL, 0.125)
    b = oracle.sum_f32(list(x), oracle.SCALE_DIV, 8.0)
    c = oracle.sum_f32(list(x / np.float32(8)))
    assert_bits_equal(a, b)
    assert_bits_equal(a, c)


# ---- exact brute force ---------------------------------------------------------

def _f32_from_fraction(q):
    """Round an exact rational to binary32, round-to-nearest-even."""
    if q == 0:
        return 0.0
    sign = -1 if q < 0 else 1
    a = abs(q)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, -126)
    ulp = Fraction(2) ** (e - 23)
    m = a / ulp
    fl = m.numerator // m.denominator
    rem = m - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (fl & 1)):
        fl += 1
    val = fl * ulp
    if val >= Fraction(2) ** 128:
        return sign * float("inf")
    return sign * float(val)


def _exact_chain(col):
    acc = Fraction(float(col[0]))
    for v in col[1:]:
        acc = Fraction(_f32_from_fraction(acc + Fraction(float(v))))
    return _f32_from_fraction(acc)


def test_f32_brute_force_exact_rationals():
    rng = np.random.default_rng(3)
    k, n = 9, 300
    # wide exponent spread so that rounding happens at every step
    x = (rng.standard_normal((k, n)) * np.exp(rng.uniform(-30, 30, (k, n)))).astype(np.float32)
    x[:, 0] = np.float32(1e-45)
    x[:, 1] = [np.float32(2.0 ** 24)] + [np.float32(1.0)] * (k - 1)
    x[:, 2] = [np.float32(1.0)] * (k - 1) + [np.float32(2.0 ** 24)]
    want = np.array([_exact_chain(x[:, i]) for i in range(n)], np.float32)
    assert_bits_equal(oracle.sum_f32(list(x)), want, "brute force")


def test_bf16_rounding_against_struct():
    # every bf16 midpoint neighbourhood: compare the RNE pack with exact rationals
    rng = np.random.default_rng(5)
    vals = rng.standard_normal(2000).astype(np.float32)
    vals[:6] = [1.00390625, 1.01171875, 1.0078125, -1.00390625, 3.3895314e38, 1e-40]
    got = oracle.np_f32_to_bf16_rne(vals)
    for v, g in zip(vals, got):
        u = struct.unpack("<I", struct.pack("<f", float(v)))[0]
        lo = u & 0xFFFF0000
        hi = lo + 0x10000
        flo = struct.unpack("<f", struct.pack("<I", lo))[0]
        fhi = struct.unpack("<f", struct.pack("<I", hi & 0xFFFFFFFF))[0]
        if np.isinf(fhi) or np.isnan(fhi):
            # top binade: the next bf16 up is the infinity encoding, whose
            # "value" for rounding purposes is 2^128
            fhi_q = Fraction(2) ** 128 * (1 if v > 0 else -1)
        else:
            fhi_q = Fraction(fhi)
        dlo = abs(Fraction(float(v)) - Fraction(flo))
        dhi = abs(fhi_q - Fraction(float(v)))
        if dlo < dhi:
            want = lo >> 16
        elif dhi < dlo:
            want = (hi >> 16) & 0xFFFF
        else:
            want = (lo >> 16) if ((lo >> 16) & 1) == 0 else (hi >> 16) & 0xFFFF
        assert int(g) == want, (v, hex(int(g)), hex(want))


# ---- known answers from the reference's benchmark --------------------------------

@pytest.mark.parametrize("k", [2, 8, 64])
def test_all_ones_kat(k):
    x = np.ones((k, 4097), np.float32)
    assert (oracle.sum_f32(list(x)) == np.float32(k)).all()
    ones_bf16 = np.full((k, 4097), 0x3F80, np.uint16)
    assert (oracle.sum_bf16(list(ones_bf16)) == oracle.np_f32_to_bf16_rne(np.full(1, k, np.float32))[0]).all()


def test_arange_kat():
    k, n = 8, 100000  # n*k < 2^24 so every partial sum is exact
    base = np.arange(n, dtype=np.float32)
    got = oracle.sum_f32([base] * k)
    assert_bits_equal(got, base * np.float32(k))


def test_max_semantics():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((5, 1000)).astype(np.float32)
    x[2, 3] = np.nan
    x[:, 4] = [-0.0, 0.0, -0.0, 0.0, -0.0]
    want = torch.amax(torch.from_numpy(x), dim=0).numpy()
    got = oracle.max_f32(list(x))
    assert np.isnan(got[3]) and np.isnan(want[3])
    m = np.ones(1000, bool)
    m[3] = m[4] = False  # sign of a zero maximum is not specified
    assert_bits_equal(got[m], want[m])
    assert got[4] == 0.0


@pytest.mark.parametrize("kind,tdt", [("f32", torch.float32), ("bf16", torch.bfloat16),
                                      ("f16", torch.float16)])
def test_max_of_every_floating_type_against_aten_amax(kind, tdt):
    # the maximum of the 2-byte types, pinned directly against the installed ATen's amax on the
    # CPU (what the reference calls, fairring/device.cc:127): NaN in any position wins, +-inf,
    # +-0 (whose sign ATen leaves unspecified), subnormals, K = 1 ... 64
    rng = np.random.default_rng(19)
    for k in (1, 2, 3, 8, 17, 64):
        n = 4000
        x = (rng.standard_normal((k, n)) * np.exp(rng.uniform(-20, 20, (k, n)))).astype(np.float32)
        x[:, 0] = np.inf
        x[:, 1] = -np.inf
        x[rng.integers(k), 2] = np.inf
        x[rng.integers(k), 3] = -np.inf
        x[rng.integers(k), 4] = np.nan                 # one NaN among finite values
        x[:, 5] = np.nan
        x[:, 6] = [(-0.0 if r % 2 else 0.0) for r in range(k)]
        x[:, 7] = -0.0
        x[:, 8] = np.float32(1e-41) * (np.arange(k) - k // 2)   # fp32 subnormals of both signs
        x[:, 9] = np.float32(6e-8) * (np.arange(k) + 1)         # fp16 subnormals
        x[rng.integers(k), 10] = np.nan
        x[(rng.integers(k) + 1) % k, 10] = np.inf      # NaN beats +inf wherever either stands
        t = torch.from_numpy(x).to(tdt)
        want_t = torch.amax(t, dim=0)
        if kind == "f32":
            got, want = oracle.reduce(kind, list(x), "max"), want_t.numpy()
            zero = want == 0
        else:
            bits = t.view(torch.int16).numpy().view(np.uint16)
            got = oracle.reduce(kind, list(bits), "max")
            want = want_t.view(torch.int16).numpy().view(np.uint16)
            zero = (want & 0x7FFF) == 0
        assert zero[6] and zero[7]
        if kind == "f32":
            assert (got[zero] == 0).all()
        else:
            assert ((got[zero] & 0x7FFF) == 0).all()
        assert_bits_equal(got[~zero], want[~zero], "%s amax K=%d" % (kind, k), half=kind == "f16")
    # exhaustively over pairs of special values and a few ordinary ones, both orders
    specials = np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, 1.0, -1.0, 65504.0, 6e-8, -6e-8,
                         1e-41, 3.0e38], np.float32)
    a, b = np.meshgrid(specials, specials)
    pair = torch.from_numpy(np.stack([a.reshape(-1), b.reshape(-1)])).to(tdt)
    want_t = torch.amax(pair, dim=0)
    if kind == "f32":
        got, want = oracle.reduce(kind, list(pair.numpy()), "max"), want_t.numpy()
        zero = want == 0
    else:
        got = oracle.reduce(kind, list(pair.view(torch.int16).numpy().view(np.uint16)), "max")
        want = want_t.view(torch.int16).numpy().view(np.uint16)
        zero = (want & 0x7FFF) == 0
    assert_bits_equal(got[~zero], want[~zero], kind + " amax of pairs", half=kind == "f16")


# ---- the other element types ----------------------------------------------------------

def test_f16_conversions_exhaustive_and_sum_vs_aten():
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float32)
    back = oracle.reduce("f16", [bits])          # K = 1: f16 -> f32 -> f16 must be the identity
    assert_bits_equal(back, bits, "f16 round trip", half=True)
    # every binary32 midpoint between neighbouring halves rounds to even, checked with numpy
    rng = np.random.default_rng(17)
    x = (rng.standard_normal((8, 50000)) * np.exp(rng.uniform(-14, 12, (8, 50000)))).astype(np.float32)
    h = x.astype(np.float16)
    got = oracle.reduce("f16", list(h.view(np.uint16)))
    want = torch.sum(torch.from_numpy(h), dim=0).numpy().view(np.uint16)   # fp32 accumulate, one RNE
    assert_bits_equal(got, want, "f16 sum", half=True)
    got = oracle.reduce("f16", list(h.view(np.uint16)), "sum", oracle.SCALE_MUL, 0.125)
    acc = h[0].astype(np.float32)
    for k in range(1, 8):
        acc = acc + h[k].astype(np.float32)
    with np.errstate(over="ignore"):
        want = (acc * np.float32(0.125)).astype(np.float16).view(np.uint16)
    assert_bits_equal(got, want, "f16 mul", half=True)
    assert vals[0x3C00] == 1.0


def test_f64_and_integer_types_vs_numpy_and_aten():
    rng = np.random.default_rng(18)
    d = rng.standard_normal((9, 20000)) * np.exp(rng.uniform(-40, 40, (9, 20000)))
    acc = d[0].copy()
    for k in range(1, 9):
        acc = acc + d[k]
    assert_bits_equal(oracle.reduce("f64", list(d)), acc, "f64 chain")
    assert_bits_equal(oracle.reduce("f64", list(d), "sum", oracle.SCALE_DIV, 9.0), acc / 9.0, "f64 div")
    t = torch.from_numpy(d)
    chain = t[0].clone()
    for k in range(1, 9):
        chain = torch.add(chain, t[k])
    assert_bits_equal(oracle.reduce("f64", list(d)), chain.numpy(), "f64 vs at::add")
    for kind, npdt, lo, hi in (("i32", np.int32, -2**31, 2**31), ("i64", np.int64, -2**63, 2**63),
                               ("u8", np.uint8, 0, 256), ("i8", np.int8, -128, 128)):
        x = rng.integers(lo, hi, (7, 5000), dtype=npdt)       # full range: sums wrap around
        with np.errstate(over="ignore"):
            want = x[0].copy()
            for k in range(1, 7):
                want = (want + x[k]).astype(npdt)
        assert (oracle.reduce(kind, list(x)) == want).all(), kind
        # ATen sums integers in int64 and casts to the output type: the same wrap-around
        tw = torch.sum(torch.from_numpy(x), dim=0).to(torch.from_numpy(x).dtype).numpy()
        assert (oracle.reduce(kind, list(x)) == tw).all(), kind + " vs aten"
        assert (oracle.reduce(kind, list(x), "max") == x.max(axis=0)).all(), kind + " max"
    m = oracle.reduce("f64", list(d), "max")
    assert (m == d.max(axis=0)).all()


# ---- DDP hook arithmetic on either side of the reduction ---------------------------------
# Pinned against the very expressions of torch's hooks
# (torch:distributed/algorithms/ddp_comm_hooks/default_hooks.py:18-93) run by the installed torch.

def _wide_f32(rng, shape):
    x = (rng.standard_normal(shape) * np.exp(rng.uniform(-30, 30, shape))).astype(np.float32)
    x.reshape(-1)[:6] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1e-42]   # special lanes, a subnormal
    return x


@pytest.mark.parametrize("world", [2, 3, 6, 7, 8, 48])
def test_pre_scale_matches_torch_allreduce_hook(world):
    rng = np.random.default_rng(300 + world)
    x = _wide_f32(rng, (world, 4099))
    # allreduce_hook: every rank runs tensor.div_(world) on its bucket, then the buckets are summed
    terms = [torch.from_numpy(r.copy()).div_(world) for r in x]
    acc = terms[0].clone()
    for t in terms[1:]:
        acc = torch.add(acc, t)
    assert_bits_equal(oracle.sum_f32(list(x), oracle.SCALE_PRE_DIV, float(world)), acc.numpy(),
                      "fp32 pre-div")
    assert_bits_equal(oracle.sum_f32(list(x), oracle.SCALE_PRE_DIV, float(world), chain=True,
                                     threads=3), acc.numpy(), "fp32 pre-div, blocked chain")
    # ATen on the GPU multiplies by the reciprocal of a scalar divisor instead
    s = np.float32(1) / np.float32(world)
    terms = [torch.from_numpy(r.copy()).mul_(torch.tensor(s)) for r in x]
    acc = terms[0].clone()
    for t in terms[1:]:
        acc = torch.add(acc, t)
    assert_bits_equal(oracle.sum_f32(list(x), oracle.SCALE_PRE_MUL, float(s)), acc.numpy(),
                      "fp32 pre-mul")
    # half types: the scaled bucket is a tensor of the half type, so every term is rounded
    for kind, dt in (("bf16", torch.bfloat16), ("f16", torch.float16)):
        h = [torch.from_numpy(r.copy()).to(dt) for r in x]
        bits = [t.view(torch.int16).numpy().view(np.uint16) for t in h]
        terms = [t.clone().div_(world) for t in h]
        acc = terms[0].float()
        for t in terms[1:]:
            acc = acc + t.float()
        want = acc.to(dt).view(torch.int16).numpy().view(np.uint16)
        got = oracle.reduce(kind, bits, "sum", oracle.SCALE_PRE_DIV, float(world))
        assert_bits_equal(got, want, kind + " pre-div", half=True)
    d = x.astype(np.float64)
    with np.errstate(all="ignore"):
        acc = d[0] / world
        for k in range(1, world):
            acc = acc + d[k] / world
    assert_bits_equal(oracle.reduce("f64", list(d), "sum", oracle.SCALE_PRE_DIV, float(world)), acc,
                      "f64 pre-div")


@pytest.mark.parametrize("world,rank", [(2, 1), (8, 3), (5, 0)])
def test_gathered_reduce_matches_torch_bucket_assembly(world, rank):
    # What DDP's reducer does ahead of the allreduce, run by the installed torch: every gradient
    # is copied to its place in the flat bucket (torch.cat lays them end to end like the bucket
    # views), multiplied by 1/world where no hook is registered (mul_out into the view), and the
    # buckets are summed in rank order.
    rng = np.random.default_rng(900 + world)
    lens = [4099, 1, 0, 2048, 3, 70001]
    n = sum(lens)
    x = _wide_f32(rng, (world, n))
    grads = [torch.from_numpy(x[rank, sum(lens[:i]):sum(lens[:i + 1])].copy()) for i in range(len(lens))]
    s = np.float32(1) / np.float32(world)
    for pre in (False, True):
        buckets = [torch.from_numpy(r.copy()) for r in x]
        buckets[rank] = torch.cat(grads)
        if pre:
            buckets = [b.mul(torch.tensor(s)) for b in buckets]
        acc = buckets[0].clone()
        for b in buckets[1:]:
            acc = torch.add(acc, b)
        contribs = [None if k == rank else x[k] for k in range(world)]
        got = oracle.gathered_reduce("f32", contribs, rank, [g.numpy() for g in grads], "sum",
                                     oracle.SCALE_PRE_MUL if pre else oracle.SCALE_NONE, float(s))
        assert_bits_equal(got, acc.numpy(), "gathered, pre-scale %s" % pre)
    # bf16 gradients: one rounding at the end of an fp32 fold, like the plain sum
    h = [torch.from_numpy(r.copy()).to(torch.bfloat16) for r in x]
    hg = [g.to(torch.bfloat16) for g in grads]
    hb = list(h)
    hb[rank] = torch.cat(hg)
    acc = hb[0].float()
    for b in hb[1:]:
        acc = acc + b.float()
    want = acc.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    bits = [None if k == rank else t.view(torch.int16).numpy().view(np.uint16) for k, t in enumerate(h)]
    got = oracle.gathered_reduce("bf16", bits, rank,
                                 [g.view(torch.int16).numpy().view(np.uint16) for g in hg])
    assert_bits_equal(got, want, "gathered bf16")


@pytest.mark.parametrize("wire,dt", [("bf16", torch.bfloat16), ("f16", torch.float16)])
@pytest.mark.parametrize("world", [1, 2, 3, 8, 64])
def test_compressed_sum_matches_torch_compress_hook(wire, dt, world):
    rng = np.random.default_rng(400 + world)
    x = _wide_f32(rng, (world, 3001))
    # _compress_hook on every rank: buffer.to(dtype).div_(world_size)
    comp = [torch.from_numpy(r.copy()).to(dt).div_(world) for r in x]
    # the allreduce of the compressed tensors: fp32 fold in rank order, one rounding
    acc = comp[0].float()
    for c in comp[1:]:
        acc = acc + c.float()
    reduced = acc.to(dt)
    # decompress: buffer.copy_(value)
    buffer = torch.from_numpy(x[0].copy())
    buffer.copy_(reduced)
    peers = [c.view(torch.int16).numpy().view(np.uint16) for c in comp]
    wire_bits = reduced.view(torch.int16).numpy().view(np.uint16)
    for raw in sorted({0, world // 2, world - 1}):
        contribs = list(peers)
        contribs[raw] = x[raw]
        got = oracle.compressed_sum(contribs, raw, wire, oracle.SCALE_DIV, float(world))
        assert_bits_equal(got, buffer.numpy(), "%s raw %d -> fp32" % (wire, raw))
        got = oracle.compressed_sum(contribs, raw, wire, oracle.SCALE_DIV, float(world),
                                    out_f32=False)
        assert_bits_equal(got, wire_bits, "%s raw %d -> wire" % (wire, raw), half=True)
    # no raw contribution: the plain reduction of the wire type, widened or not
    got = oracle.compressed_sum(peers, -1, wire, out_f32=False)
    assert_bits_equal(got, oracle.reduce(wire, peers), wire + " all peers", half=True)
    assert_bits_equal(got, wire_bits, wire + " all peers vs torch", half=True)


def test_compressed_sum_bf16_numpy_twin():
    rng = np.random.default_rng(55)
    x = _wide_f32(rng, (5, 2000))
    peers = [oracle.np_f32_to_bf16_rne(r) for r in x]
    s = np.float32(1) / np.float32(5)
    with np.errstate(all="ignore"):
        own = oracle.np_bf16_to_f32(oracle.np_f32_to_bf16_rne(x[3]))
        own = oracle.np_bf16_to_f32(oracle.np_f32_to_bf16_rne(own * s))
        acc = oracle.np_bf16_to_f32(peers[0])
        for k in range(1, 5):
            acc = acc + (own if k == 3 else oracle.np_bf16_to_f32(peers[k]))
        want = oracle.np_bf16_to_f32(oracle.np_f32_to_bf16_rne(acc))
    contribs = list(peers)
    contribs[3] = x[3]
    assert_bits_equal(oracle.compressed_sum(contribs, 3, "bf16", oracle.SCALE_MUL, float(s)), want)


# ---- layout and slicing ---------------------------------------------------------------

MiB = 1024 * 1024


def test_compute_layout_known_answers():
    assert oracle.compute_layout(50 * MiB, MiB, 16, 1, 1) == dict(
        slot=3276784, slice=3276784, padding_slots=16, staging_slots=16)
    assert oracle.compute_layout(50 * MiB, MiB, 16, 8, 1) == dict(
        slot=3276672, slice=3276672, padding_slots=16, staging_slots=16)
    assert oracle.compute_layout(50 * MiB, MiB, 2, 1, 1) == dict(
        slot=26214384, slice=26214384, padding_slots=2, staging_slots=2)
    lay = oracle.compute_layout(50 * MiB, MiB, 16, 4, 8)
    assert lay == dict(slot=0, slice=2 ** 63 - 1, padding_slots=4096, staging_slots=0)
    with pytest.raises(ValueError):
        oracle.compute_layout(50 * MiB, 64, 16, 1, 1)   # 64/8 = 8 padding slots < 16
    with pytest.raises(ValueError):
        oracle.compute_layout(100, MiB, 16, 1, 1)        # padding alone exceeds the pool


def test_compute_layout_hand_formula():
    # independent evaluation of the D == 1 branch with Python integers
    for total, par, m in [(50 * MiB, 16, 1), (123456789, 7, 3), (MiB, 1, 64)]:
        unit = m * 8
        slot = ((total - 2 * par * unit) // par) // unit * unit
        lay = oracle.compute_layout(total, MiB, par, m, 1)
        assert lay["slot"] == slot and lay["slice"] == slot
        assert lay["staging_slots"] == par and lay["padding_slots"] == par


def test_slicing_known_answers():
    S = 25 * MiB
    assert oracle.num_slices(1_370_000_000, S, 4) == 210
    assert oracle.slice_bounds(1_370_000_000, S, 4, 209) == (209 * 6_553_600, 297_600)
    assert oracle.num_slices(1_300_000_000, S, 2) == 100
    assert oracle.slice_bounds(1_300_000_000, S, 2, 99) == (99 * 13_107_200, 2_387_200)
    assert oracle.num_slices(0, S, 4) == 0
    assert oracle.num_slices(6_553_600, S, 4) == 1
    assert oracle.num_slices(6_553_601, S, 4) == 2
    assert oracle.slice_bounds(6_553_601, S, 4, 1) == (6_553_600, 1)
    assert oracle.lib().orc_readme_layout(50 * MiB, 25 * MiB) == 2


def test_slices_tile_the_tensor():
    for numel, sb, es in [(1000, 96, 4), (1001, 96, 4), (5, 8, 2), (12345, 1000, 2)]:
        n = oracle.num_slices(numel, sb, es)
        pos = 0
        for i in range(n):
            off, ln = oracle.slice_bounds(numel, sb, es, i)
            assert off == pos and 0 < ln <= sb // es
            pos += ln
        assert pos == numel
