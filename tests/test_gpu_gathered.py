"""GPU parity of the launches over several pieces (frg_reduce_pieces) and of the allreduce
with one contribution given piecewise (frg_allreduce_gathered: a bucket's own gradients read
from where autograd left them), through the C ABI, against the CPU oracle. Bit-exact.
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
KINDS = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def _print_case(*a):
    print("[case]", *a, flush=True)


def host_values(kind, rng, shape):
    """Random values of the kind as the oracle takes them (fp32, or uint16 bit patterns)."""
    x = (rng.standard_normal(shape) * 0.01).astype(np.float32)
    if kind == "f32":
        return x
    if kind == "bf16":
        return oracle.np_f32_to_bf16_rne(x)
    return x.astype(np.float16).view(np.uint16)


def to_gpu(kind, a, skew=0):
    """A GPU tensor holding `a`, starting `skew` elements past a 16-byte boundary."""
    a = np.ascontiguousarray(a)
    if kind == "f32":
        t = torch.from_numpy(a)
    else:
        t = torch.from_numpy(a.view(np.int16)).view(KINDS[kind])
    buf = torch.empty(a.size + skew + 8, dtype=t.dtype, device=DEV)
    buf[skew:skew + a.size].copy_(t)
    return buf[skew:skew + a.size]


def from_gpu(kind, t):
    if kind == "f32":
        return t.cpu().numpy()
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


SCALES = [("none", fa.SCALE_NONE, oracle.SCALE_NONE, lambda k: 1.0),
          ("mul", fa.SCALE_MUL, oracle.SCALE_MUL, lambda k: 1.0 / k),
          ("div", fa.SCALE_DIV, oracle.SCALE_DIV, lambda k: float(k)),
          ("pre_mul", fa.SCALE_PRE_MUL, oracle.SCALE_PRE_MUL, lambda k: float(np.float32(1) / np.float32(k))),
          ("pre_div", fa.SCALE_PRE_DIV, oracle.SCALE_PRE_DIV, lambda k: float(k))]


@pytest.mark.parametrize("kind", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("k", [1, 2, 3, 4, 8, 9, 16, 17])
def test_reduce_pieces_vs_oracle(kind, k):
    rng = np.random.default_rng(77 * k + len(kind))
    sizes = [1, 3, 4, 5, 0, 255, 1024, 4099, 262147, 7, 1_500_003, 8, 16, 2048, 33]
    for name, mode, omode, scale_of in SCALES:
        _print_case("pieces", kind, k, name)
        host, pieces, outs = [], [], []
        for i, n in enumerate(sizes):
            x = host_values(kind, rng, (k, n))
            # every third piece has one contribution off the others' position within 16 bytes
            # (a launch of its own); every fourth is reduced in place
            skews = [(1 if (i % 3 == 2 and j == k - 1) else 0) for j in range(k)]
            cs = [to_gpu(kind, x[j], skews[j]) for j in range(k)]
            out = cs[0] if i % 4 == 3 else torch.empty(n + 8, dtype=KINDS[kind], device=DEV)[:n]
            host.append(x)
            pieces.append((out, cs))
            outs.append(out)
        fa.reduce_pieces(pieces, scale_mode=mode, scale=scale_of(k))
        torch.cuda.synchronize()
        for i, x in enumerate(host):
            want = oracle.reduce(kind, list(x), "sum", omode, scale_of(k))
            assert_bits_equal(from_gpu(kind, outs[i]), want, "%s k=%d piece %d (%d el) %s" % (
                kind, k, i, sizes[i], name), half=kind == "f16")


@pytest.mark.parametrize("kind", ["f32", "bf16"])
@pytest.mark.parametrize("k,scale", [(1, "none"), (3, "mul"), (5, "mul"), (7, "pre_mul"), (8, "div"),
                                     (8, "pre_div"), (4, "div"), (9, "mul"), (16, "none")])
def test_reduce_pieces_full_tables_at_every_group_size(kind, k, scale):
    # 60 pieces that all fit the segmented kernel: launches with the table full (24 pieces up
    # to 8 contributions, 12 beyond), also at group sizes and scales that have no variant of
    # their own and share the one that takes the number of contributions at run time.
    _print_case("pieces, full tables", kind, k, scale)
    rng = np.random.default_rng(1000 * k + len(scale))
    name, mode, omode, scale_of = [sc for sc in SCALES if sc[0] == scale][0]
    per16 = 4 if kind == "f32" else 8
    host = [host_values(kind, rng, (k, per16 * int(n))) for n in rng.integers(1, 700, size=60)]
    pieces = [(torch.empty(x.shape[1], dtype=KINDS[kind], device=DEV), [to_gpu(kind, r) for r in x])
              for x in host]
    fa.reduce_pieces(pieces, scale_mode=mode, scale=scale_of(k))
    torch.cuda.synchronize()
    for i, ((out, _), x) in enumerate(zip(pieces, host)):
        want = oracle.reduce(kind, list(x), "sum", omode, scale_of(k))
        assert_bits_equal(from_gpu(kind, out), want, "piece %d" % i)


@pytest.mark.parametrize("seed", range(4))
def test_reduce_pieces_random_cases(seed):
    # Random element type, number of contributions (1 to 20: beyond 16 every piece is a
    # launch of its own), scale, number of pieces (1 to 70), and per piece a random length,
    # a random place of every buffer within 16 bytes (tidy pieces share launches, the others
    # go alone) and in place or not. Against the oracle.
    rng = np.random.default_rng(9500 + seed)
    for case in range(6):
        kind = ["f32", "bf16", "f16"][int(rng.integers(0, 3))]
        per16 = 4 if kind == "f32" else 8
        k = int(rng.integers(1, 21))
        name, mode, omode, scale_of = SCALES[int(rng.integers(0, 5))]
        count = int(rng.integers(1, 71))
        _print_case("pieces, random", seed, case, kind, k, name, count)
        host, pieces = [], []
        for i in range(count):
            n = int(rng.integers(0, 1 << int(rng.integers(1, 16))))
            x = host_values(kind, rng, (k, n))
            tidy = rng.integers(0, 4) > 0
            cs = [to_gpu(kind, x[j], 0 if tidy else int(rng.integers(0, per16))) for j in range(k)]
            if rng.integers(0, 4) == 0:
                out = cs[int(rng.integers(0, k))]
            else:
                out = torch.zeros(n + 16, dtype=KINDS[kind], device=DEV)
                sk = 0 if tidy else int(rng.integers(0, per16))
                out = out[sk:sk + n]
            host.append(x)
            pieces.append((out, cs))
        fa.reduce_pieces(pieces, scale_mode=mode, scale=scale_of(k))
        torch.cuda.synchronize()
        for i, ((out, _), x) in enumerate(zip(pieces, host)):
            want = oracle.reduce(kind, list(x), "sum", omode, scale_of(k))
            assert_bits_equal(from_gpu(kind, out), want, "seed %d case %d piece %d" % (seed, case, i),
                              half=kind == "f16")


def test_reduce_pieces_many_small_tensors_and_other_kinds():
    # more pieces than one launch takes; MAX and int32 go piece by piece through the plain kernel
    _print_case("pieces many")
    rng = np.random.default_rng(5)
    k = 8
    host = [(rng.standard_normal((k, n)) * 0.01).astype(np.float32)
            for n in rng.integers(1, 3000, size=100)]
    pieces = [(torch.empty(x.shape[1], device=DEV), [to_gpu("f32", r) for r in x]) for x in host]
    fa.reduce_pieces(pieces, scale_mode=fa.SCALE_MUL, scale=0.125)
    torch.cuda.synchronize()
    for (out, _), x in zip(pieces, host):
        assert_bits_equal(out.cpu().numpy(), oracle.sum_f32(list(x), oracle.SCALE_MUL, 0.125))
    fa.reduce_pieces(pieces, op=fa.MAX)
    torch.cuda.synchronize()
    for (out, _), x in zip(pieces, host):
        assert_bits_equal(out.cpu().numpy(), oracle.max_f32(list(x)))
    ih = [rng.integers(-2**31, 2**31, size=(3, n), dtype=np.int64).astype(np.int32) for n in (5, 4099)]
    ip = [(torch.empty(x.shape[1], dtype=torch.int32, device=DEV),
           [torch.from_numpy(r.copy()).to(DEV) for r in x]) for x in ih]
    fa.reduce_pieces(ip)
    torch.cuda.synchronize()
    for (out, _), x in zip(ip, ih):
        assert (out.cpu().numpy() == oracle.reduce("i32", list(x))).all()


def bucket_case(kind, rng, k, g, lens, skew_every=0):
    """Peers' buckets, this rank's gradients as tensors of their own, and the host copies."""
    n = int(sum(lens))
    x = host_values(kind, rng, (k, n))
    peers = [None if j == g else to_gpu(kind, x[j]) for j in range(k)]
    segs, off = [], 0
    for i, ln in enumerate(lens):
        skew = 1 if skew_every and i % skew_every == 1 else 0
        segs.append(to_gpu(kind, x[g, off:off + ln], skew))
        off += ln
    return x, peers, segs, n


LAYER = [2048 * 2048, 2048, 2048, 2048 * 512, 2048, 1, 3, 4096, 0, 2048 * 64 + 5, 16]


@pytest.mark.parametrize("kind", ["f32", "bf16"])
@pytest.mark.parametrize("k,g", [(8, 0), (8, 5), (2, 1), (3, 2), (16, 7)])
def test_allreduce_gathered_vs_oracle(kind, k, g):
    rng = np.random.default_rng(31 * k + g)
    dev = fa.DeviceFairring(0, slice_size_in_bytes=25 * MiB, max_memory_allocated_in_bytes=50 * MiB)
    for name, mode, omode, scale_of in SCALES[:4]:
        _print_case("gathered", kind, k, g, name)
        x, peers, segs, n = bucket_case(kind, rng, k, g, LAYER)
        out = torch.empty(n, dtype=KINDS[kind], device=DEV)
        dev.allreduce_gathered(out, peers, g, segs, scale_mode=mode, scale=scale_of(k)).wait()
        want = oracle.reduce(kind, list(x), "sum", omode, scale_of(k))
        assert_bits_equal(from_gpu(kind, out), want, "%s k=%d g=%d %s" % (kind, k, g, name))
    assert dev.progress()["segmented_launches"] > 0
    dev.close()


def test_allreduce_gathered_misaligned_segments_other_reductions_and_the_copy_it_replaces():
    rng = np.random.default_rng(12)
    dev = fa.DeviceFairring(0)
    # gradients that start off a 16-byte boundary, odd lengths ahead of big tensors
    lens = [5, 300001, 1, 1 << 20, 7, 2048, 2048, 33, 1 << 18]
    for kind, k, g in (("f32", 8, 3), ("f16", 4, 0), ("bf16", 8, 7)):
        _print_case("gathered misaligned", kind, k)
        x, peers, segs, n = bucket_case(kind, rng, k, g, lens, skew_every=2)
        out = torch.empty(n, dtype=KINDS[kind], device=DEV)
        dev.allreduce_gathered(out, peers, g, segs, scale_mode=fa.SCALE_MUL, scale=1.0 / k).wait()
        want = oracle.reduce(kind, list(x), "sum", oracle.SCALE_MUL, 1.0 / k)
        assert_bits_equal(from_gpu(kind, out), want, kind, half=kind == "f16")
        # the same bits as copying every gradient into the bucket and reducing that in place
        bucket = torch.cat(segs)
        full = [bucket if j == g else peers[j] for j in range(k)]
        dev.allreduce(bucket, full, scale_mode=fa.SCALE_MUL, scale=1.0 / k).wait()
        assert torch.equal(bucket.view(torch.int16 if kind != "f32" else torch.int32),
                           out.view(torch.int16 if kind != "f32" else torch.int32))
    # more contributions than the segmented kernel takes, and MAX: plain launches per segment
    _print_case("gathered k=20, max")
    x, peers, segs, n = bucket_case("f32", rng, 20, 4, [4099, 1, 70000, 2048])
    out = torch.empty(n, device=DEV)
    dev.allreduce_gathered(out, peers, 4, segs, scale_mode=fa.SCALE_DIV, scale=20.0).wait()
    assert_bits_equal(out.cpu().numpy(), oracle.sum_f32(list(x), oracle.SCALE_DIV, 20.0))
    dev.allreduce_gathered(out, peers, 4, segs, op=fa.MAX).wait()
    assert_bits_equal(out.cpu().numpy(), oracle.max_f32(list(x)))
    # 70 bf16 contributions: a chain of launches per segment, one rounding
    _print_case("gathered k=70 bf16")
    x, peers, segs, n = bucket_case("bf16", rng, 70, 69, [4099, 3, 30000])
    out = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    dev.allreduce_gathered(out, peers, 69, segs).wait()
    assert_bits_equal(from_gpu("bf16", out), oracle.sum_bf16(list(x)))
    # contract
    with pytest.raises(fa.FairringError):
        dev.allreduce_gathered(out, peers, 69, segs[:-1])
    dev.close()


@pytest.mark.parametrize("seed", range(4))
def test_allreduce_gathered_random_layouts(seed):
    # Random gradient tensors (one to forty, from a few elements to a few MiB, some empty),
    # every buffer at a random place within 16 bytes, random element type, group size, rank
    # and scale: segmented launches of many pieces, single pieces as plain launches, pieces
    # whose pointers disagree modulo 16. Against the oracle.
    rng = np.random.default_rng(8000 + seed)
    dev = fa.DeviceFairring(0, slice_size_in_bytes=25 * MiB, max_memory_allocated_in_bytes=50 * MiB)
    try:
        for case in range(8):
            kind = ["f32", "bf16", "f16"][int(rng.integers(0, 3))]
            per16 = 4 if kind == "f32" else 8
            k = int(rng.integers(1, 18))
            g = int(rng.integers(0, k))
            name, mode, omode, scale_of = SCALES[int(rng.integers(0, 5))]
            tidy = bool(rng.integers(0, 2))
            lens = []
            for i in range(int(rng.integers(1, 41))):
                ln = per16 * int(rng.integers(1, 1 << int(rng.integers(2, 19 if i < 3 else 14))))
                if not tidy and rng.integers(0, 3) == 0:
                    ln += int(rng.integers(-per16 + 1, per16))
                if rng.integers(0, 10) == 0:
                    ln = 0
                lens.append(max(ln, 0))
            if sum(lens) == 0:
                lens[0] = 5
            n = int(sum(lens))
            _print_case("gathered, random", seed, case, kind, k, g, name, tidy, lens)
            x = host_values(kind, rng, (k, n))
            peers = [None if j == g else to_gpu(kind, x[j], 0 if tidy else int(rng.integers(0, per16)))
                     for j in range(k)]
            segs, off = [], 0
            for ln in lens:
                segs.append(to_gpu(kind, x[g, off:off + ln], 0 if tidy else int(rng.integers(0, per16))))
                off += ln
            oskew = 0 if tidy else int(rng.integers(0, per16))
            out = torch.zeros(n + 16, dtype=KINDS[kind], device=DEV)[oskew:oskew + n]
            dev.allreduce_gathered(out, peers, g, segs, scale_mode=mode, scale=scale_of(k)).wait()
            want = oracle.reduce(kind, list(x), "sum", omode, scale_of(k))
            assert_bits_equal(from_gpu(kind, out), want, "seed %d case %d" % (seed, case),
                              half=kind == "f16")
        assert dev.progress()["segmented_launches"] > 0
    finally:
        dev.close()


def test_allreduce_gathered_waits_for_the_gradients_and_orders_what_follows():
    # the gradients are still being written on the caller's stream when the operation is
    # submitted; and an operation that overwrites a gradient afterwards runs behind it
    _print_case("gathered ordering")
    k, g = 8, 2
    n_big = 8 * MiB
    dev = fa.DeviceFairring(0)
    peers = [None if j == g else torch.full((2 * n_big,), float(j), device=DEV) for j in range(k)]
    for _ in range(3):
        grads = [torch.zeros(n_big, device=DEV), torch.zeros(n_big, device=DEV)]
        out = torch.empty(2 * n_big, device=DEV)
        busy = torch.empty(64 * MiB, device=DEV)
        for _ in range(6):
            busy.normal_()                      # keeps the stream busy for a few milliseconds
        grads[0].fill_(100.0)
        grads[1].fill_(200.0)
        w = dev.allreduce_gathered(out, peers, g, grads)
        # overwrites the first gradient: must run after the operation above has read it
        ones = [torch.ones(n_big, device=DEV) for _ in range(2)]
        w2 = dev.allreduce(grads[0], ones)
        w.wait()
        w2.wait()
        torch.cuda.synchronize()
        rest = float(sum(j for j in range(k) if j != g))
        assert float(out[:n_big].min()) == rest + 100.0 == float(out[:n_big].max())
        assert float(out[n_big:].min()) == rest + 200.0 == float(out[n_big:].max())
        assert float(grads[0].min()) == 2.0 == float(grads[0].max())
    dev.close()


# ---- the compression hooks' reduction with the raw contribution in tensors of its own ---------

# ten tensors that all start where a lane's group of 8 elements does: a launch reads up to
# eight of them through its table
ALIGNED_LAYER = [2048 * 2048, 2048, 2048, 2048 * 512, 2048, 8, 4096, 16, 2048 * 64 + 8, 24]


@pytest.mark.parametrize("wire,tdt", [("bf16", torch.bfloat16), ("f16", torch.float16)])
@pytest.mark.parametrize("k,g", [(8, 0), (8, 5), (2, 1), (4, 3), (17, 9), (1, 0)])
def test_allreduce_compressed_gathered_through_the_table(wire, tdt, k, g):
    # Layer sizes that are multiples of 8 (and the allocator's alignment): the bucket is cut as
    # an assembled one would be, and each launch reads its raw term from up to eight gradient
    # tensors by a table in its arguments: two launches for these ten tensors. With the bucket
    # and the peers 4 elements into a group of 8 (the groups then start 4 elements into every
    # tensor) no launch takes the table, and every tensor is a launch of its own: ten.
    rng = np.random.default_rng(171 * k + g)
    dev = fa.DeviceFairring(0, slice_size_in_bytes=25 * MiB, max_memory_allocated_in_bytes=50 * MiB)
    try:
        lens = ALIGNED_LAYER
        n = int(sum(lens))
        for name, mode, omode, scale_of in SCALES[:3]:
            for skew in (0, 4):
                _print_case("compressed gathered, table", wire, k, g, name, skew)
                x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
                bits = oracle.np_f32_to_bf16_rne(x) if wire == "bf16" else x.astype(np.float16).view(np.uint16)
                host = [bits[j] for j in range(k)]
                host[g] = x[g]
                peers = [None if j == g else to_gpu(wire, bits[j], skew) for j in range(k)]
                segs, off = [], 0
                for ln in lens:
                    segs.append(to_gpu("f32", x[g, off:off + ln], skew))
                    off += ln
                s = scale_of(k) if name != "mul" else float(np.float32(1) / np.float32(k))
                out = torch.full((n + 16,), 7.0, device=DEV)[skew:skew + n]
                before = dev.progress()["launches"]
                dev.allreduce_compressed(out, peers, g, scale_mode=mode, scale=s, wire_dtype=tdt,
                                         segments=segs).wait()
                launches = dev.progress()["launches"] - before
                if skew == 0:
                    # (17 contributions: launches of about 80 MB cut the bucket in three)
                    assert launches == (2 if k <= 8 else 4)
                elif k > 1:
                    assert launches >= 10
                else:
                    assert launches == 2     # no peers: 16 bytes off is still a 16-byte boundary
                want = oracle.compressed_sum(host, g, wire, omode, s)
                assert_bits_equal(out.cpu().numpy(), want, "%s k=%d g=%d %s skew %d" % (wire, k, g, name, skew))
    finally:
        dev.close()


@pytest.mark.parametrize("wire,tdt", [("bf16", torch.bfloat16), ("f16", torch.float16)])
@pytest.mark.parametrize("k,g", [(8, 2), (4, 0), (5, 4)])
def test_allreduce_compressed_gathered_table_with_scalar_ends(wire, tdt, k, g):
    # The peers' wire tensors 8 bytes past a 16-byte boundary: a launch then has a head of 4
    # scalar elements, its groups of 8 start 4 elements in, and the gradient tensors fit the
    # table when they start there too (the first one 4 elements longer than a multiple of 8);
    # 3 elements are left behind the last group. The scalars at both ends are reduced by lanes
    # of one block that sit in different tensors.
    rng = np.random.default_rng(191 * k + g)
    lens = [2048 * 2048 + 4, 2048, 2048 * 512, 8, 2048 * 64 + 8 + 3]
    n = int(sum(lens))
    dev = fa.DeviceFairring(0, slice_size_in_bytes=25 * MiB, max_memory_allocated_in_bytes=50 * MiB)
    try:
        for name, mode, omode, scale_of in SCALES[:2]:
            _print_case("compressed gathered, table, scalar ends", wire, k, g, name)
            x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
            bits = oracle.np_f32_to_bf16_rne(x) if wire == "bf16" else x.astype(np.float16).view(np.uint16)
            host = [bits[j] for j in range(k)]
            host[g] = x[g]
            peers = [None if j == g else to_gpu(wire, bits[j], 4) for j in range(k)]
            segs, off = [], 0
            for ln in lens:
                segs.append(to_gpu("f32", x[g, off:off + ln], 0))
                off += ln
            s = scale_of(k) if name != "mul" else float(np.float32(1) / np.float32(k))
            out = torch.full((n + 16,), 7.0, device=DEV)[4:4 + n]
            before = dev.progress()["launches"]
            dev.allreduce_compressed(out, peers, g, scale_mode=mode, scale=s, wire_dtype=tdt,
                                     segments=segs).wait()
            assert dev.progress()["launches"] - before == 1
            want = oracle.compressed_sum(host, g, wire, omode, s)
            assert_bits_equal(out.cpu().numpy(), want, "%s k=%d g=%d %s" % (wire, k, g, name))
    finally:
        dev.close()


@pytest.mark.parametrize("wire,tdt", [("bf16", torch.bfloat16), ("f16", torch.float16)])
@pytest.mark.parametrize("k,g", [(8, 0), (8, 5), (2, 1), (4, 3), (17, 9)])
def test_allreduce_compressed_gathered_vs_oracle(wire, tdt, k, g):
    # The raw fp32 contribution (rank g) as the gradient tensors of a layer, the peers'
    # contributions as wire tensors of the bucket's length, the fp32 bucket written once:
    # the oracle's compressed sum over the concatenated gradients, and the bits of the
    # one-pass reduction over an assembled bucket (frg_allreduce_compressed in place).
    rng = np.random.default_rng(131 * k + g)
    dev = fa.DeviceFairring(0, slice_size_in_bytes=25 * MiB, max_memory_allocated_in_bytes=50 * MiB)
    try:
        for name, mode, omode, scale_of in SCALES[:3]:
            _print_case("compressed gathered", wire, k, g, name)
            lens = LAYER if name != "div" else [2048 * 2048 * 2, 5, 2048 * 512 + 3]   # the last: large tensors, odd ends
            n = int(sum(lens))
            x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
            bits = oracle.np_f32_to_bf16_rne(x) if wire == "bf16" else x.astype(np.float16).view(np.uint16)
            host = [bits[j] for j in range(k)]
            host[g] = x[g]
            peers = [None if j == g else to_gpu(wire, bits[j]) for j in range(k)]
            segs, off = [], 0
            for ln in lens:
                segs.append(to_gpu("f32", x[g, off:off + ln]))
                off += ln
            s = scale_of(k) if name != "mul" else float(np.float32(1) / np.float32(k))
            out = torch.full((n,), 7.0, device=DEV)
            dev.allreduce_compressed(out, peers, g, scale_mode=mode, scale=s, wire_dtype=tdt,
                                     segments=segs).wait()
            want = oracle.compressed_sum(host, g, wire, omode, s)
            assert_bits_equal(out.cpu().numpy(), want, "%s k=%d g=%d %s" % (wire, k, g, name))
            # the assembled bucket, reduced in place
            bucket = to_gpu("f32", x[g])
            contribs = list(peers)
            contribs[g] = bucket
            dev.allreduce_compressed(bucket, contribs, g, scale_mode=mode, scale=s, wire_dtype=tdt).wait()
            assert bool(torch.equal(bucket.view(torch.int32), out.view(torch.int32)))
    finally:
        dev.close()


@pytest.mark.parametrize("seed", range(6))
def test_allreduce_compressed_gathered_random_layouts(seed):
    # Random gradient tensors (between one and twelve, mostly multiples of 8 elements long,
    # some not, some empty), random places of every buffer within 16 bytes, random group size,
    # rank, wire type, scale and output type: launches that take their tensors through the
    # table (with and without scalar ends, whole tiles and tiles that straddle tensors) and
    # launches that fall back to a tensor each. Against the oracle, and for the launch count
    # only that the result does not depend on it.
    rng = np.random.default_rng(7000 + seed)
    dev = fa.DeviceFairring(0, slice_size_in_bytes=25 * MiB, max_memory_allocated_in_bytes=50 * MiB)
    through_table = tensor_each = 0
    try:
        for case in range(8):
            k = int(rng.integers(1, 10))
            g = int(rng.integers(0, k))
            wire, tdt = [("bf16", torch.bfloat16), ("f16", torch.float16)][int(rng.integers(0, 2))]
            name, mode, omode, scale_of = SCALES[int(rng.integers(0, 3))]
            out_f32 = bool(rng.integers(0, 4) > 0)
            pieces = int(rng.integers(1, 13))
            tidy = bool(rng.integers(0, 3) > 0)          # two cases in three: everything lines up
            base = int(rng.choice([0, 4])) if tidy else 0
            lens = []
            for i in range(pieces):
                ln = 8 * int(rng.integers(1, 1 << int(rng.integers(4, 17))))
                if i == 0:
                    ln += base
                if not tidy and rng.integers(0, 3) == 0:
                    ln += int(rng.integers(-7, 8))
                if rng.integers(0, 10) == 0:
                    ln = 0 if i > 0 else ln
                lens.append(max(ln, 0))
            lens[-1] += int(rng.integers(0, 8))          # scalars behind the last group
            n = int(sum(lens))
            wskew = base if tidy else int(rng.integers(0, 8))
            oskew = (base % 4 if out_f32 else base) if tidy else int(rng.integers(0, 4))
            _print_case("compressed gathered, random", seed, case, wire, k, g, name, out_f32, tidy, lens)
            x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
            bits = oracle.np_f32_to_bf16_rne(x) if wire == "bf16" else x.astype(np.float16).view(np.uint16)
            host = [bits[j] for j in range(k)]
            host[g] = x[g]
            peers = [None if j == g else to_gpu(wire, bits[j], wskew) for j in range(k)]
            segs, off = [], 0
            for ln in lens:
                segs.append(to_gpu("f32", x[g, off:off + ln], 0 if tidy else int(rng.integers(0, 4))))
                off += ln
            s = scale_of(k) if name != "mul" else float(np.float32(1) / np.float32(k))
            if out_f32:
                out = torch.full((n + 16,), 7.0, device=DEV)[oskew:oskew + n]
            else:
                out = torch.zeros(n + 16, dtype=tdt, device=DEV)[oskew:oskew + n]
            before = dev.progress()["launches"]
            dev.allreduce_compressed(out, peers, g, scale_mode=mode, scale=s, wire_dtype=tdt,
                                     segments=segs).wait()
            launches = dev.progress()["launches"] - before
            filled = sum(1 for ln in lens if ln > 0)
            through_table += int(filled > 1 and launches < filled)
            tensor_each += int(filled > 1 and launches >= filled)
            want = oracle.compressed_sum(host, g, wire, omode, s, out_f32=out_f32)
            got = out.cpu().numpy() if out_f32 else from_gpu(wire, out)
            assert_bits_equal(got, want, "seed %d case %d" % (seed, case))
        print("through the table: %d, a tensor each: %d" % (through_table, tensor_each), flush=True)
        assert through_table >= 1 and tensor_each >= 1     # both routes, for every seed here
    finally:
        dev.close()


def test_allreduce_compressed_gathered_wire_output_and_contract():
    _print_case("compressed gathered: wire output, contract")
    rng = np.random.default_rng(9)
    k, g = 4, 2
    lens = [4099, 0, 262147, 1]
    n = int(sum(lens))
    x = (rng.standard_normal((k, n)) * 0.01).astype(np.float32)
    bits = oracle.np_f32_to_bf16_rne(x)
    host = [bits[j] for j in range(k)]
    host[g] = x[g]
    peers = [None if j == g else to_gpu("bf16", bits[j]) for j in range(k)]
    segs, off = [], 0
    for ln in lens:
        segs.append(to_gpu("f32", x[g, off:off + ln]))
        off += ln
    dev = fa.DeviceFairring(0)
    try:
        out = torch.empty(n, dtype=torch.bfloat16, device=DEV)
        dev.allreduce_compressed(out, peers, g, wire_dtype=torch.bfloat16, segments=segs).wait()
        want = oracle.compressed_sum(host, g, "bf16", oracle.SCALE_NONE, 1.0, out_f32=False)
        assert_bits_equal(from_gpu("bf16", out), want, "wire output")
        with pytest.raises(fa.FairringError):                       # lengths must add up
            dev.allreduce_compressed(torch.empty(n, device=DEV), peers, g, wire_dtype=torch.bfloat16,
                                     segments=segs[:-1])
        with pytest.raises(fa.FairringError):                       # segments are fp32
            dev.allreduce_compressed(torch.empty(n, device=DEV), peers, g, wire_dtype=torch.bfloat16,
                                     segments=[s.to(torch.bfloat16) for s in segs])
    finally:
        dev.close()
