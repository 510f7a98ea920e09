"""Seeded random walk over the argument space of the reduction, through the C
ABI against the CPU oracle (bit-exact): element type x op x scale mode x K x
length x pointer alignment x in-place or not x one launch or the slice
pipeline with a random slice size, stream count and launch size. Every case
prints its parameters before it touches the GPU."""
import zlib

import numpy as np
import pytest
import torch

import oracle
from conftest import assert_bits_equal

pytestmark = pytest.mark.gpu

fa = pytest.importorskip("fairring_amd")

DEV = "cuda:0"
KINDS = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16,
         "f64": torch.float64, "i32": torch.int32, "i64": torch.int64, "u8": torch.uint8,
         "i8": torch.int8}
SCALES = {"none": (fa.SCALE_NONE, oracle.SCALE_NONE), "mul": (fa.SCALE_MUL, oracle.SCALE_MUL),
          "div": (fa.SCALE_DIV, oracle.SCALE_DIV), "premul": (fa.SCALE_PRE_MUL, oracle.SCALE_PRE_MUL),
          "prediv": (fa.SCALE_PRE_DIV, oracle.SCALE_PRE_DIV)}


def to_gpu(a, tdt):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if tdt in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).to(DEV).view(tdt)
    return t.to(DEV)


def to_np(t):
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


def random_values(kind, rng, k, n):
    if kind in ("f32", "bf16", "f16", "f64"):
        spread = {"f32": 20, "bf16": 20, "f16": 6, "f64": 40}[kind]
        x = rng.standard_normal((k, n)) * np.exp(rng.uniform(-spread, spread, (k, n)))
        if n >= 4:
            x[rng.integers(k), 0] = np.inf
            x[rng.integers(k), 1] = np.nan
            x[:, 2] = 0.0
            x[rng.integers(k), 2] = -0.0
        if kind == "f64":
            return x
        x = x.astype(np.float32)
        if kind == "f32":
            return x
        if kind == "bf16":
            return oracle.np_f32_to_bf16_rne(x).reshape(k, n)
        with np.errstate(over="ignore"):
            return x.astype(np.float16).view(np.uint16)
    info = np.iinfo(oracle.TYPES[kind][0])
    return rng.integers(info.min, int(info.max) + 1, (k, n), dtype=oracle.TYPES[kind][0])


def draw_case(seed):
    rng = np.random.default_rng(seed)
    kind = list(KINDS)[rng.integers(len(KINDS))]
    floating = oracle.TYPES[kind][1]
    op = "max" if rng.random() < 0.25 else "sum"
    scale = "none"
    if floating and op == "sum":
        scale = list(SCALES)[rng.integers(len(SCALES))]
    pipeline = rng.random() < 0.5
    k = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 12, 16, 23, 33, 64]))
    if pipeline and rng.random() < 0.2:
        k = int(rng.integers(65, 140))          # chained launches with a carried term
    n = int(rng.choice([1, 2, 15, 16, 17, 255, 1000, 4096, 4099, 65537, 300_011, 1_048_577]))
    if k > 32:
        n = min(n, 65537)
    shift = int(rng.integers(0, 9))             # elements off the allocation's start
    in_place = rng.random() < 0.3
    return dict(seed=seed, kind=kind, op=op, scale=scale, pipeline=pipeline, k=k, n=n,
                shift=shift, in_place=in_place,
                slice_bytes=int(rng.choice([8 * 1024, 64 * 1024, 1024 * 1024])),
                streams=int(rng.integers(1, 4)),
                launch_div=int(rng.choice([1, 2, 3])))


@pytest.mark.parametrize("seed", range(160))
def test_random_case(seed):
    c = draw_case(zlib.crc32(b"fairring-matrix") + seed)
    print("[case]", c, flush=True)
    kind, tdt, k, n, shift = c["kind"], KINDS[c["kind"]], c["k"], c["n"], c["shift"]
    rng = np.random.default_rng(c["seed"] + 1)
    x = random_values(kind, rng, k, n + shift)
    big = [to_gpu(r, tdt) for r in x]
    views = [b[shift:] for b in big]
    in_place_at = int(rng.integers(k)) if c["in_place"] else -1
    if in_place_at >= 0:
        out = views[in_place_at]
        guard = None
    else:
        guard = torch.zeros(n + shift + 8, dtype=tdt, device=DEV)
        out = guard[shift:shift + n]
    fmode, omode = SCALES[c["scale"]]
    sval = 1.0
    if c["scale"] in ("mul", "premul"):
        sval = float(np.float32(1) / np.float32(k))
    elif c["scale"] in ("div", "prediv"):
        sval = float(k)
    fop = fa.SUM if c["op"] == "sum" else fa.MAX
    if c["pipeline"]:
        dev = fa.DeviceFairring(0, slice_size_in_bytes=c["slice_bytes"],
                                max_memory_allocated_in_bytes=2 * c["slice_bytes"],
                                num_reduce_streams=c["streams"],
                                max_launch_bytes=max(16, c["slice_bytes"] // c["launch_div"]))
        dev.allreduce(out, views, op=fop, scale_mode=fmode, scale=sval).wait()
        dev.close()
    else:
        fa.reduce_slice(out, views, op=fop, scale_mode=fmode, scale=sval)
        torch.cuda.synchronize()
    if oracle.TYPES[kind][1] and c["op"] == "sum":
        want = oracle.reduce(kind, list(x[:, shift:]), "sum", omode, sval)
    else:
        want = oracle.reduce(kind, list(x[:, shift:]), c["op"])
    got = to_np(out)
    if c["op"] == "max" and kind in ("f32", "bf16", "f16", "f64"):
        # the sign of a zero maximum is not specified (at::amax: +0 and -0 compare equal)
        zero = (want == 0) if kind in ("f32", "f64") else ((want & 0x7FFF) == 0)
        assert ((got[zero] == 0) if kind in ("f32", "f64") else ((got[zero] & 0x7FFF) == 0)).all()
        got, want = got[~zero], want[~zero]
    assert_bits_equal(got, want, str(c), half=kind == "f16")
    if guard is not None:   # nothing outside the output range was written
        assert int(torch.count_nonzero(guard[:shift].view(torch.uint8))) == 0
        assert int(torch.count_nonzero(guard[shift + n:].view(torch.uint8))) == 0


def draw_host_case(seed):
    rng = np.random.default_rng(seed)
    kind = list(KINDS)[rng.integers(len(KINDS))]
    floating = oracle.TYPES[kind][1]
    op = "max" if rng.random() < 0.25 else "sum"
    scale = "none"
    if floating and op == "sum":
        scale = ["none", "mul", "div"][rng.integers(3)]
    return dict(seed=seed, kind=kind, op=op, scale=scale, k=int(rng.integers(1, 14)),
                n=int(rng.choice([1, 17, 4099, 65537, 300_011])),
                slots=int(rng.integers(1, 7)), carry=bool(rng.random() < 0.4),
                slice_bytes=int(rng.choice([16 * 1024, 256 * 1024, 1024 * 1024])),
                copy_streams=int(rng.integers(1, 4)))


@pytest.mark.parametrize("seed", range(60))
def test_random_host_staged_case(seed):
    # contributions in pinned host memory, staged through 1 to 6 slots and folded in order
    c = draw_host_case(zlib.crc32(b"fairring-host-matrix") + seed)
    print("[case]", c, flush=True)
    kind, tdt, k, n = c["kind"], KINDS[c["kind"]], c["k"], c["n"]
    rng = np.random.default_rng(c["seed"] + 1)
    x = random_values(kind, rng, k, n)

    def pinned(a):
        t = torch.from_numpy(np.ascontiguousarray(a))
        if tdt in (torch.float16, torch.bfloat16):
            t = t.view(torch.int16).view(tdt)
        return t.pin_memory()

    fmode, omode = SCALES[c["scale"]]
    sval = {"none": 1.0, "mul": float(np.float32(1) / np.float32(k)), "div": float(k)}[c["scale"]]
    fop = fa.SUM if c["op"] == "sum" else fa.MAX
    dev = fa.DeviceFairring(0, slice_size_in_bytes=c["slice_bytes"],
                            max_memory_allocated_in_bytes=c["slots"] * c["slice_bytes"],
                            num_copy_streams=c["copy_streams"])
    if c["carry"]:
        out = to_gpu(x[0], tdt)
        dev.allreduce_host(out, [pinned(r) for r in x[1:]], op=fop, scale_mode=fmode, scale=sval,
                           carry=True).wait()
    else:
        out = torch.empty(n, dtype=tdt, device=DEV)
        dev.allreduce_host(out, [pinned(r) for r in x], op=fop, scale_mode=fmode,
                           scale=sval).wait()
    dev.close()
    if oracle.TYPES[kind][1] and c["op"] == "sum":
        want = oracle.reduce(kind, list(x), "sum", omode, sval)
    else:
        want = oracle.reduce(kind, list(x), c["op"])
    got = to_np(out)
    if c["op"] == "max" and kind in ("f32", "bf16", "f16", "f64"):
        zero = (want == 0) if kind in ("f32", "f64") else ((want & 0x7FFF) == 0)
        got, want = got[~zero], want[~zero]
    assert_bits_equal(got, want, str(c), half=kind == "f16")


def draw_compressed_case(seed):
    rng = np.random.default_rng(seed)
    k = int(rng.choice([1, 2, 3, 5, 8, 9, 16, 31, 64]))
    return dict(seed=seed, wire=["bf16", "f16"][rng.integers(2)], k=k,
                raw=int(rng.integers(-1, k)),
                n=int(rng.choice([1, 7, 8, 9, 1000, 4099, 65537, 300_011, 1_048_577])),
                shift=int(rng.integers(0, 9)), out_f32=bool(rng.random() < 0.7),
                in_place=bool(rng.random() < 0.5),
                mode=["none", "mul", "div"][rng.integers(3)], pipeline=bool(rng.random() < 0.5),
                slice_bytes=int(rng.choice([8 * 1024, 64 * 1024, 1024 * 1024])),
                streams=int(rng.integers(1, 4)), launch_div=int(rng.choice([1, 2, 3])))


@pytest.mark.parametrize("seed", range(100))
def test_random_compressed_case(seed):
    # the reduction with a compression hook folded in: raw fp32 bucket at a random rank
    c = draw_compressed_case(zlib.crc32(b"fairring-compressed-matrix") + seed)
    print("[case]", c, flush=True)
    wire, tdt, k, n, shift, raw = c["wire"], KINDS[c["wire"]], c["k"], c["n"], c["shift"], c["raw"]
    rng = np.random.default_rng(c["seed"] + 1)
    xf = random_values("f32", rng, k, n + shift)
    if wire == "bf16":
        bits = oracle.np_f32_to_bf16_rne(xf).reshape(xf.shape)
    else:
        with np.errstate(over="ignore"):
            bits = xf.astype(np.float16).view(np.uint16)
    contribs = [to_gpu(bits[i], tdt)[shift:] for i in range(k)]
    contribs_np = [bits[i, shift:] for i in range(k)]
    if raw >= 0:
        contribs[raw] = to_gpu(xf[raw], torch.float32)[shift:]
        contribs_np[raw] = xf[raw, shift:]
    out_dt = torch.float32 if c["out_f32"] else tdt
    # a float32 output may be the raw bucket itself, a wire-type output any peer's tensor
    if c["out_f32"]:
        alias = [raw] if raw >= 0 else []
    else:
        alias = [i for i in range(k) if i != raw]
    if c["in_place"] and alias:
        out = contribs[alias[int(rng.integers(len(alias)))]]
    else:
        out = torch.empty(n + shift, dtype=out_dt, device=DEV)[shift:]
    fmode, omode = SCALES[c["mode"]]
    sval = {"none": 1.0, "mul": float(np.float32(1) / np.float32(k)), "div": float(k)}[c["mode"]]
    if c["pipeline"]:
        dev = fa.DeviceFairring(0, slice_size_in_bytes=c["slice_bytes"],
                                max_memory_allocated_in_bytes=2 * c["slice_bytes"],
                                num_reduce_streams=c["streams"],
                                max_launch_bytes=max(16, c["slice_bytes"] // c["launch_div"]))
        dev.allreduce_compressed(out, contribs, raw, scale_mode=fmode, scale=sval,
                                 wire_dtype=tdt).wait()
        dev.close()
    else:
        fa.reduce_slice_compressed(out, contribs, raw, scale_mode=fmode, scale=sval, wire_dtype=tdt)
        torch.cuda.synchronize()
    want = oracle.compressed_sum(contribs_np, raw, wire, omode, sval, out_f32=c["out_f32"])
    assert_bits_equal(to_np(out), want, str(c), half=(wire == "f16" and not c["out_f32"]))
