"""The one-launch entry points under HIP graph capture: frg_reduce_slice and
frg_reduce_slice_compressed allocate nothing, record no event and clear no
memory, so a launch-bound loop over many small buckets can be captured once
and replayed. Every replay is compared bit for bit with the eager result on
the same inputs, with the program's own eager work and synchronisations
between the replays."""
import pytest
import torch

import fairring_amd as fa

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
K = 8


def same_bits(a, b):
    if a.dtype in (torch.float32, torch.int32):
        return bool(torch.equal(a.view(torch.int32), b.view(torch.int32)))
    return bool(torch.equal(a.view(torch.int16), b.view(torch.int16)))


def fill(xs, gen, scale=0.01):
    for x in xs:
        x.copy_((torch.randn(x.numel(), device=DEV, generator=gen) * scale).to(x.dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_captured_loop_over_small_buckets_replays_bit_exactly(dtype):
    print("[case] graph capture of reduce_slice", dtype, flush=True)
    sizes = [1, 7, 1024, 4099, 65536, 262144, 300007, 1 << 20] * 2     # 16 buckets, ragged ones too
    gen = torch.Generator(device=DEV)
    gen.manual_seed(77)
    xs = [[torch.empty(n, dtype=dtype, device=DEV) for _ in range(K)] for n in sizes]
    outs = [torch.zeros(n, dtype=dtype, device=DEV) for n in sizes]
    eager = [torch.zeros(n, dtype=dtype, device=DEV) for n in sizes]

    def loop(dst):
        for o, c in zip(dst, xs):
            fa.reduce_slice(o, c, scale_mode=fa.SCALE_MUL, scale=0.125)

    for c in xs:
        fill(c, gen)
    loop(eager)                       # loads the kernels before anything is captured
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        loop(outs)
    for replay in range(4):
        for c in xs:                  # new contents at the captured addresses
            fill(c, gen)
        loop(eager)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, (o, e) in enumerate(zip(outs, eager)):
            assert same_bits(o, e), "replay %d bucket %d (%d elements)" % (replay, i, sizes[i])
        for o in outs:
            o.zero_()
    # the first bucket against plain arithmetic, so that eager and replay are not wrong together
    want = xs[2][0].float()
    for x in xs[2][1:]:
        want = want + x.float()
    assert same_bits(eager[2], (want * 0.125).to(dtype))


def test_captured_compressed_reduction_replays_bit_exactly():
    print("[case] graph capture of reduce_slice_compressed", flush=True)
    sizes = [5, 4099, 262144, 1 << 20]
    gen = torch.Generator(device=DEV)
    gen.manual_seed(78)
    own = [torch.empty(n, device=DEV) for n in sizes]
    keep = [torch.empty(n, device=DEV) for n in sizes]
    peers = [[torch.empty(n, dtype=torch.bfloat16, device=DEV) for _ in range(K - 1)] for n in sizes]
    eager = [torch.empty(n, device=DEV) for n in sizes]

    def loop(dst):
        for o, b, p in zip(dst, own, peers):
            fa.reduce_slice_compressed(o, [b] + p, raw_index=0, scale_mode=fa.SCALE_MUL, scale=0.125)

    def refill():
        fill(keep, gen)
        for p in peers:
            fill(p, gen, 0.00125)

    refill()
    for b, k in zip(own, keep):
        b.copy_(k)
    loop(eager)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        loop(own)                     # in place, as the hook runs it: the bucket receives the result
    for replay in range(3):
        refill()
        for b, k in zip(own, keep):
            b.copy_(k)
        loop(eager)                   # reads the buckets, writes elsewhere
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, (b, e) in enumerate(zip(own, eager)):
            assert same_bits(b, e), "replay %d bucket %d" % (replay, i)


def test_the_pipeline_refuses_a_capturing_stream():
    # the pipeline launches from its own thread on its own streams, which a capture of the
    # caller's stream cannot record: it says so instead of splitting the work across the graph
    print("[case] pipeline under capture", flush=True)
    n = 100_000
    xs = [torch.ones(n, device=DEV) for _ in range(K)]
    out = torch.zeros(n, device=DEV)
    dev = fa.DeviceFairring(0)
    dev.allreduce(out, xs).wait()
    assert bool((out == K).all())
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        with pytest.raises(fa.FairringError, match="captured"):
            dev.allreduce(out, xs)
        fa.reduce_slice(out, xs, scale_mode=fa.SCALE_MUL, scale=0.5)   # this one may be captured
    out.zero_()
    graph.replay()
    torch.cuda.synchronize()
    assert bool((out == K * 0.5).all())
    dev.allreduce(out, xs).wait()        # and the context works as before afterwards
    assert bool((out == K).all())
    dev.close()
