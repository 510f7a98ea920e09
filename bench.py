#!/usr/bin/env python3
"""Benchmark of the K-way gradient-slice reduction on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2]

Default workload c2 (the configuration the metric is quoted on): K = 8
simulated rank contributions of a 1.37 G-element fp32 gradient, N(0, sigma =
0.01) from fixed seeds, reduced in contribution order with the divide-by-8
fused into the store, processed as 25 MiB slices (210 of them, the last
297,600 elements) into one output buffer. A step is one pass over the whole
gradient; inputs are resident in HBM before the timed region starts. Bytes
counted are the algorithmic ones: (K + 1) * numel * elsize per step.

Other workloads (the remaining configurations of the benchmark definition, for the record):
  c4    bf16, K = 8 x 1.3 G elements, fp32 accumulate, RNE store, fused /8
  c3    K = 64 contributions of one 25 MiB fp32 slice staged from pinned host
        memory with hipMemcpyAsync, overlapped with the accumulate kernel
  c5    DDP backward stream: the 1.37 G gradient as 25 MiB buckets (first one
        1 MiB) released in reverse order, one allreduce call per bucket
  c5pg  the same bucket stream through the drop-in surface: one
        _fairring.ProcessGroup.allreduce per bucket (group of 8, 7 simulated
        peers resident on the GPU, in place, completion through the future,
        every work waited for at the end of the step)
  c5sep the bucket stream as DistributedDataParallel lays it out: 48 buckets of
        25 MiB, every bucket and every peer's copy of it an allocation of its
        own, one _fairring.ProcessGroup.allreduce per bucket
  gather the c5sep layout with the bucket's own contribution still in six
        gradient tensors of its own per bucket, through
        ProcessGroup._allreduce_from_grads: the copy into the bucket is part of
        the reduction; the record also holds the rate of copy-then-allreduce
        on the same data
  copy  K = 1 (a plain copy of known size), the calibration for HBM counters
  placement  the c2 reduction on 400 M elements at six placements of its buffers
        in one process (diagnostic, prints its own line)
  hook  torch's bf16 compression hook folded into the reduction: own fp32
        gradient compressed in registers + 7 peers' bf16 tensors, result
        decompressed in place (22 algorithmic bytes per element)

Prints one JSON line with the whole-job GB/s, the roofline of the reduction
kernel (algorithmic bytes per launch / average launch duration from HIP events
on the kernel's own stream) and a CPU baseline timed on this host's cores. The
default run (c2) then measures the other workloads as well, briefly, and adds
them to the same line under "configs" (--no-extra-configs leaves them out).

The default warm-up is 120 steps (0.9 s), the default timed region 100 steps.
A process that starts right after another one has released tens of GB of
device memory runs about 4 % slower while the device deals with that memory
(about a second per 40 GiB; 6,608 -> 6,750 GB/s one second into such a
process), and a short timed region at the very start of the process sits
inside that window. For the same reason nothing is handed back to the driver
between the workloads of one run.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MiB = 1024 * 1024
HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E peak


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=120)
    ap.add_argument("--workload", default="c2",
                    choices=["c2", "c3", "c4", "c5", "c5pg", "c5sep", "gather", "copy", "hook",
                             "smallops", "placement"])
    ap.add_argument("--extras", default="c5,c5pg,c4,c5sep,gather,hook,c3",
                    help="default workload only: the workloads measured afterwards, in this order")
    ap.add_argument("--no-extra-configs", action="store_true",
                    help="default workload only: do not measure the other workloads afterwards")
    ap.add_argument("--numel", type=int, default=0, help="override the workload's element count")
    ap.add_argument("--k", type=int, default=0, help="override the number of contributions")
    ap.add_argument("--slice-bytes", type=int, default=25 * MiB)
    ap.add_argument("--total-memory", type=int, default=50 * MiB)
    ap.add_argument("--streams", type=int, default=0, help="reduce streams (0 = library default)")
    ap.add_argument("--launch-bytes", type=int, default=0,
                    help="bytes of one contribution per launch (0 = library default, -1 = slice)")
    ap.add_argument("--copy-streams", type=int, default=0, help="host-staged path (0 = default)")
    ap.add_argument("--blocks-per-cu", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-slices", type=int, default=16)
    return ap.parse_args()


def oracle_slice(oracle, host, dtype, k, scale):
    cores = os.cpu_count() or 1
    if dtype == "f32":
        mode = oracle.SCALE_MUL if scale else oracle.SCALE_NONE
        return oracle.sum_f32(host, mode, 1.0 / k if scale else 1.0, threads=cores)
    mode = oracle.SCALE_MUL if scale else oracle.SCALE_NONE
    return oracle.sum_bf16(host, mode, 1.0 / k if scale else 1.0, threads=cores)


def to_host(np, torch, t):
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


def check_parity(oracle, np, torch, xs, out, numel, slice_elems, k, dtype, scale):
    """Bit-compare the first, a middle and the ragged last slice with the oracle
    fed the very bytes the GPU read."""
    n_slices = (numel + slice_elems - 1) // slice_elems
    checked = []
    for idx in sorted({0, n_slices // 2, n_slices - 1}):
        lo = idx * slice_elems
        hi = min(numel, lo + slice_elems)
        host = [to_host(np, torch, x[lo:hi]) for x in xs]
        want = oracle_slice(oracle, host, dtype, k, scale)
        got = to_host(np, torch, out[lo:hi])
        if dtype == "f32":
            ok = (got.view(np.uint32) == want.view(np.uint32)).all()
        else:
            ok = (got == want).all()
        if not ok:
            raise SystemExit("parity FAILED on slice %d" % idx)
        checked.append(idx)
    return checked


TORCH_PASSES = 150   # timed passes of the CPU baseline (about ten seconds of CPU work in all)
ORACLE_PASSES = 30


def cpu_baseline_sample(xs, slice_elems, n_sample):
    """The first `n_sample` slices of every contribution, copied back from the GPU."""
    return [[x[i * slice_elems:(i + 1) * slice_elems].cpu() for x in xs]
            for i in range(n_sample)]


def cpu_baseline(oracle, np, torch, host, slice_elems, k, dtype):
    """The contract's reduction on this host's cores: torch's at::add chain
    (acc = x0; acc += xk; acc /= K; bf16: fp32 accumulator, one final cast) over
    the distinct 25 MiB slices in `host` (cpu_baseline_sample); 3 warm-up and
    TORCH_PASSES timed passes, median. The repository's C restatement (OpenMP) is timed
    beside it. GB/s uses the same algorithmic-bytes formula as the GPU figure."""
    n_sample = len(host)
    threads = torch.get_num_threads()
    xs = host[0]
    acc = torch.empty(slice_elems, dtype=torch.float32)
    res = torch.empty(slice_elems, dtype=xs[0].dtype)

    def one_pass():
        for sl in host:
            acc.copy_(sl[0])
            for c in sl[1:]:
                acc.add_(c)
            acc.div_(float(k))
            if dtype != "f32":
                res.copy_(acc)

    for _ in range(3):
        one_pass()
    times = []
    for _ in range(TORCH_PASSES):
        t0 = time.perf_counter()
        one_pass()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    elsize = 4 if dtype == "f32" else 2
    algo_bytes = (k + 1) * slice_elems * elsize * n_sample
    torch_gbps = algo_bytes / med / 1e9

    cores = os.cpu_count() or 1
    hnp = [[to_host(np, torch, c) for c in sl] for sl in host]
    fn = oracle.sum_f32 if dtype == "f32" else oracle.sum_bf16
    kw = dict(chain=True) if dtype == "f32" else {}
    for sl in hnp[:2]:
        fn(sl, oracle.SCALE_DIV, float(k), threads=cores, **kw)
    times = []
    for _ in range(ORACLE_PASSES):
        t0 = time.perf_counter()
        for sl in hnp:
            fn(sl, oracle.SCALE_DIV, float(k), threads=cores, **kw)
        times.append(time.perf_counter() - t0)
    c_gbps = algo_bytes / sorted(times)[len(times) // 2] / 1e9
    return {
        "value": round(torch_gbps, 2), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": "%d distinct 25 MiB slices x K=%d %s, torch CPU at::add chain + div, median of "
                  "%d passes, %d torch threads of %d host cpus" % (n_sample, k, dtype, TORCH_PASSES,
                                                                    threads, cores),
        "c_oracle_gbps": round(c_gbps, 2), "c_oracle_threads": cores,
    }


def synth(torch, numel, k, dtype, seed0):
    g = torch.Generator(device="cuda:0")
    xs = []
    for r in range(k):
        g.manual_seed(seed0 + r)
        t = torch.empty(numel, dtype=torch.float32, device="cuda:0").normal_(0.0, 0.01,
                                                                             generator=g)
        xs.append(t if dtype == "f32" else t.to(torch.bfloat16))
        del t
    return xs


def union_length(intervals):
    """Total length of the union of (begin, end) intervals."""
    total, cur_b, cur_e = 0.0, None, None
    for b, e in sorted(intervals):
        if cur_e is None or b > cur_e:
            if cur_e is not None:
                total += cur_e - cur_b
            cur_b, cur_e = b, e
        else:
            cur_e = max(cur_e, e)
    if cur_e is not None:
        total += cur_e - cur_b
    return total


LAUNCH_QUANTUM_BYTES = 4096


def launch_elems(args, op_elems, slice_elems, elsize, k=8, compressed_default=0):
    """Elements of the commonest launch of an operation over `op_elems` elements.
    With a launch size asked for (or the compressed reduction's default,
    `compressed_default`), the pipeline cuts the tensor into launches of that size
    on 4 KiB boundaries from its start, the last one up to one and a half times
    as long; a negative size means one launch per slice. Otherwise the partition
    is the library's own (frg_plan_launches: launches of whole rounds of their
    grid from 4 contributions on)."""
    lb = args.launch_bytes or compressed_default
    if lb == 0:
        import collections

        import fairring_amd as fa
        sizes = collections.Counter(n for n, _ in fa.plan_launches(k, op_elems, elsize))
        return sizes.most_common(1)[0][0] if sizes else 0
    if lb < 0:
        return min(slice_elems, op_elems)
    max_elems = (lb - lb % 16) // elsize
    quantum = LAUNCH_QUANTUM_BYTES // elsize
    per = max_elems // quantum * quantum
    if per < quantum:
        lanes = 16 // elsize
        per = -(-max_elems // lanes) * lanes
    return per if 2 * op_elems > 3 * per else op_elems


def roofline_from_records(recs, bytes_per_elem, full_launch_elems, how):
    """Roofline of the reduction kernel from HIP-event records on its streams.
    Launches on the two reduce streams overlap on purpose, so a launch's
    duration alone understates the kernel: while two launches run, each sees
    half the bandwidth. The kernel's achieved rate is the algorithmic bytes of
    the recorded launches divided by the time during which at least one of them
    was running (the union of the recorded intervals); avg_launch_us and
    concurrency (sum of durations / union) are reported beside it, so that
    achieved = launch_bytes * concurrency / avg_launch. launch_bytes is the
    mean over the recorded launches (a bucket stream's launches are cut from
    runs of buckets, so they are not all of the planned size of a lone
    operation, which is reported as launch_elems)."""
    durs = [r[1] - r[0] for r in recs]
    launches = sum(r[5] for r in recs)
    elems = sum(r[2] for r in recs)
    busy_ms = union_length([(r[0], r[1]) for r in recs])
    achieved = elems * bytes_per_elem / (busy_ms * 1e-3) / 1e9
    return {
        "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
        "launch_bytes": int(round(elems * bytes_per_elem / max(launches, 1))),
        "launch_elems": full_launch_elems,
        "avg_launch_us": round(sum(durs) / launches * 1e3, 3), "launches_timed": launches,
        "concurrency": round(sum(durs) / busy_ms, 3),
        "streams_used": len({r[4] for r in recs}),
        "how": how,
    }


SPAN_HOW = ("HIP events on each reduce stream over the timed region: one before its first launch "
            "of the region, one after its last (launches on a stream run back to back); achieved "
            "= algorithmic bytes of those launches / union of the two spans")
LAUNCH_HOW = ("HIP events taking begin/end of every dispatch on its own stream, in a separate "
              "pass after the timed region; achieved = algorithmic bytes / union of the intervals")


def timed(torch, dev, steps, warmup, step, spans=True):
    """W untimed steps, then exactly `steps` timed ones between synchronisations.
    With spans, one HIP event per reduce stream is recorded at the start of the
    timed region and one at its end, on the streams the kernel runs on."""
    for _ in range(warmup):
        step(dev).wait()
    dev.synchronize()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    if spans:
        dev.profile_mark()
    w = None
    for _ in range(steps):
        w = step(dev)
    if spans:
        dev.profile_mark()
    w.wait()
    dev.synchronize()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    recs = dev.launch_records() if spans else None
    return elapsed, recs


def per_launch_pass(fa, args, run_steps):
    """A separate pass with every launch timed by its own dispatch timestamps."""
    dev1 = fa.DeviceFairring(0, max_memory_allocated_in_bytes=args.total_memory,
                             slice_size_in_bytes=args.slice_bytes,
                             num_reduce_streams=args.streams,
                             max_launch_bytes=args.launch_bytes,
                             num_copy_streams=args.copy_streams)
    run_steps(dev1).wait()
    dev1.synchronize()
    dev1.set_profiling(True)
    for _ in range(max(1, min(args.steps, 5))):
        run_steps(dev1)
    recs = dev1.launch_records()
    dev1.set_profiling(False)
    dev1.close()
    return recs


def run_resident(args, np, torch, fa, oracle, dtype, keep=None):
    """c2 / c4 / copy: device-resident contributions, one allreduce per step."""
    elsize = 4 if dtype == "f32" else 2
    if args.workload == "copy":
        k, numel, scale = args.k or 1, args.numel or 1_370_000_000, False
    elif dtype == "f32":
        k, numel, scale = args.k or 8, args.numel or 1_370_000_000, True
    else:
        k, numel, scale = args.k or 8, args.numel or 1_300_000_000, True
    slice_elems = args.slice_bytes // elsize
    n_slices = (numel + slice_elems - 1) // slice_elems
    dev = fa.DeviceFairring(0, max_memory_allocated_in_bytes=args.total_memory,
                            slice_size_in_bytes=args.slice_bytes,
                            num_reduce_streams=args.streams,
                            max_launch_bytes=args.launch_bytes)
    xs = synth(torch, numel, k, dtype, 20240)
    out = torch.empty(numel, dtype=xs[0].dtype, device="cuda:0")
    torch.cuda.synchronize()
    mode = fa.SCALE_MUL if scale else fa.SCALE_NONE

    def step(d):
        return d.allreduce(out, xs, scale_mode=mode, scale=1.0 / k)

    elapsed, recs = timed(torch, dev, args.steps, args.warmup, step)
    step_bytes = (k + 1) * numel * elsize
    value = step_bytes * args.steps / elapsed / 1e9
    roof = roofline_from_records(recs, (k + 1) * elsize,
                                 launch_elems(args, numel, slice_elems, elsize, k),
                                 SPAN_HOW)
    roof["kernel"] = "ksumKernel<%s, SUM, K=%d>" % ("F32Vec" if dtype == "f32" else "Bf16Vec", k)
    step(dev).wait()
    checked = check_parity(oracle, np, torch, xs, out, numel, slice_elems, k, dtype, scale)
    # and every element against the at::add chain itself, run by torch on the GPU
    chain = xs[0].float() if dtype != "f32" else xs[0].clone()
    for x in xs[1:]:
        chain.add_(x.float() if dtype != "f32" else x)
    if scale:
        chain.mul_(1.0 / k)
    same = torch.equal(out.view(torch.int32 if dtype == "f32" else torch.int16),
                       (chain if dtype == "f32" else chain.to(torch.bfloat16)).view(
                           torch.int32 if dtype == "f32" else torch.int16))
    del chain
    if not same:
        raise SystemExit("parity FAILED against the at::add chain on the GPU")
    checked = "%s; every element equal to torch's at::add chain on the GPU" % checked
    layout = dev.layout
    dev.close()
    name = {"c2": "configs[1]", "c4": "configs[3]",
            "copy": "calibration copy"}[args.workload]
    cfg = {
        "workload": "K=%d contributions x %d %s elements, %d slices of %d B, %s, one output "
                    "buffer (%s)" % (k, numel, dtype, n_slices, args.slice_bytes,
                                     "fused x1/%d" % k if scale else "no scale", name),
        "k": k, "numel": numel, "slice_bytes": args.slice_bytes,
        "staging_total_bytes": args.total_memory, "layout": layout,
        "reduce_streams": args.streams or "default",
        "launch_bytes_per_contribution": args.launch_bytes or "default",
    }
    # The CPU baseline is timed by the caller, after every GPU measurement of the
    # run: the GPU idles while the host computes, and drops its clocks.
    base = None
    if not args.no_cpu_baseline and args.workload != "copy":
        sample = cpu_baseline_sample(xs, slice_elems, min(args.cpu_slices, max(1, n_slices - 1)))
        base = lambda: cpu_baseline(oracle, np, torch, sample, slice_elems, k, dtype)  # noqa: E731
    if keep is not None:
        keep.extend([xs, out])
    return value, elapsed, cfg, roof, checked, base, dtype


def _capi_lib():
    from fairring_amd import _capi
    return _capi.lib()


def run_c3(args, np, torch, fa, oracle):
    """Server-side accumulation: K = 64 contributions of one 25 MiB fp32 slice in
    pinned host memory, staged through the pool and folded in order."""
    k, numel = args.k or 64, args.numel or 6_553_600
    g = torch.Generator(device="cuda:0")
    hs = []
    for r in range(k):
        g.manual_seed(3300 + r)
        t = torch.empty(numel, dtype=torch.float32).pin_memory()
        t.copy_(torch.empty(numel, device="cuda:0").normal_(0.0, 0.01, generator=g))
        hs.append(t)
    torch.cuda.synchronize()
    out = torch.empty(numel, dtype=torch.float32, device="cuda:0")
    dev = fa.DeviceFairring(0, max_memory_allocated_in_bytes=args.total_memory,
                            slice_size_in_bytes=args.slice_bytes,
                            num_reduce_streams=args.streams,
                            max_launch_bytes=args.launch_bytes,
                            num_copy_streams=args.copy_streams)

    def step(d):
        return d.allreduce_host(out, hs, scale_mode=fa.SCALE_MUL, scale=1.0 / k)

    elapsed, _ = timed(torch, dev, args.steps, args.warmup, step, spans=False)
    step_bytes = (k + 1) * numel * 4
    value = step_bytes * args.steps / elapsed / 1e9
    link = k * numel * 4 * args.steps / elapsed / 1e9
    slots = dev.layout["staging_slots"]
    batch = max(1, slots // max(1, len(dev._external_streams(_capi_lib().frg_get_copy_streams))))
    # What the link gives to bare copies in this run: hipMemcpyAsync (torch's non-blocking
    # copy_ from pinned memory is that call) of the same pinned buffers into two device
    # buffers of a slice's size, on the pipeline's own copy streams in turn, nothing else running.
    copy_streams = dev._external_streams(_capi_lib().frg_get_copy_streams)
    land = [torch.empty(numel, dtype=torch.float32, device="cuda:0") for _ in copy_streams]

    def bare_copies(streams, rounds):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(rounds):
            for i, h in enumerate(hs):
                with torch.cuda.stream(streams[i % len(streams)]):
                    land[i % len(streams)].copy_(h, non_blocking=True)
        torch.cuda.synchronize()
        return k * numel * 4 * rounds / (time.perf_counter() - t0) / 1e9

    bare_copies(copy_streams, 1)
    ceiling = max(bare_copies(copy_streams, 2), bare_copies(copy_streams[:1], 2))
    # the accumulate kernel of a batch reads `batch` staged slots and `out`, writes `out`
    recs = per_launch_pass(fa, args, step)
    recs = [r for r in recs if r[3] == batch]
    hbm = roofline_from_records(recs, (batch + 2) * 4, numel, LAUNCH_HOW)
    hbm["kernel"] = "ksumKernel<F32Vec, SUM, carry, K=%d>" % batch
    roof = {
        "bound": "host_link", "achieved": round(link, 2), "peak": round(ceiling, 2),
        "nominal": 64.0, "unit": "GB/s", "frac": round(link / ceiling, 4), "traffic": None,
        "how": "achieved: bytes of the K contributions crossing the host link per second of the "
               "timed region; peak: bare hipMemcpyAsync of the same pinned buffers on the same copy "
               "streams in this run (best of both streams in turn and one alone); nominal: PCIe "
               "Gen5 x16 per direction",
        "kernel": hbm["kernel"],
        "hbm": {key: hbm[key] for key in ("achieved", "peak", "frac", "launch_bytes",
                                          "avg_launch_us", "launches_timed")},
    }
    step(dev).wait()
    want = oracle.sum_f32([h.numpy() for h in hs], oracle.SCALE_MUL, 1.0 / k,
                          threads=os.cpu_count() or 1)
    got = out.cpu().numpy()
    if not (got.view(np.uint32) == want.view(np.uint32)).all():
        raise SystemExit("parity FAILED (c3)")
    layout = dev.layout
    dev.close()
    cfg = {
        "workload": "K=%d pinned-host contributions of one %d-element fp32 slice, staged with "
                    "hipMemcpyAsync through %d slots, fused x1/%d (configs[2])" % (
                        k, numel, slots, k),
        "k": k, "numel": numel, "layout": layout, "host_link_GBps": round(link, 2),
        "bound": "host link (PCIe): every contribution crosses it once",
    }
    return value, elapsed, cfg, roof, ["whole slice"], None, "f32"


def ddp_buckets(numel, bucket_elems, first_elems):
    """Buckets in the order DDP releases them: reverse parameter order, so from
    the end of the flat gradient towards its start; the first one is small."""
    spans = []
    hi = numel
    size = first_elems
    while hi > 0:
        lo = max(0, hi - size)
        spans.append((lo, hi))
        hi = lo
        size = bucket_elems
    return spans


def run_c5(args, np, torch, fa, oracle, shared=None):
    k, numel = args.k or 8, args.numel or 1_370_000_000
    slice_elems = args.slice_bytes // 4
    spans = ddp_buckets(numel, slice_elems, MiB // 4)
    dev = fa.DeviceFairring(0, max_memory_allocated_in_bytes=args.total_memory,
                            slice_size_in_bytes=args.slice_bytes,
                            num_reduce_streams=args.streams,
                            max_launch_bytes=args.launch_bytes)
    if shared is not None:   # the inputs of the c2 run (same seeds), still resident
        xs, out = shared
    else:
        xs = synth(torch, numel, k, "f32", 20240)
        out = torch.empty(numel, dtype=torch.float32, device="cuda:0")
    views = [(out[lo:hi], [x[lo:hi] for x in xs]) for lo, hi in spans]
    torch.cuda.synchronize()
    prepared = {}

    class Last:
        def __init__(self, works):
            self.works = works

        def wait(self):
            for w in self.works:
                w.wait()

    def step(d):
        # one allreduce call per bucket, in release order; the calls are marshalled once
        if id(d) not in prepared:
            prepared[id(d)] = [d.prepare(o, cs, scale_mode=fa.SCALE_MUL, scale=1.0 / k)
                               for o, cs in views]
        return Last([submit() for submit in prepared[id(d)]])

    elapsed, recs = timed(torch, dev, args.steps, args.warmup, step)
    step_bytes = (k + 1) * numel * 4
    value = step_bytes * args.steps / elapsed / 1e9
    roof = roofline_from_records(recs, (k + 1) * 4,
                                 launch_elems(args, slice_elems, slice_elems, 4, k), SPAN_HOW)
    roof["kernel"] = "ksumKernel<F32Vec, SUM, K=%d>" % k
    step(dev).wait()
    checked = check_parity(oracle, np, torch, xs, out, numel, slice_elems, k, "f32", True)
    layout = dev.layout
    dev.close()
    cfg = {
        "workload": "DDP backward stream: %d fp32 elements as %d buckets (first %d B, then %d B) "
                    "released from the end of the gradient to its start, K=%d contributions per "
                    "bucket, one allreduce call per bucket, fused x1/%d (configs[4])" % (
                        numel, len(spans), MiB, args.slice_bytes, k, k),
        "k": k, "numel": numel, "buckets": len(spans), "staging_total_bytes": args.total_memory,
        "layout": layout, "reduce_streams": args.streams or "default",
    }
    return value, elapsed, cfg, roof, checked, None, "f32"


def run_c5pg(args, np, torch, fa, oracle, shared=None):
    """The DDP bucket stream of c5 through the surface the reference exposes: one
    `_fairring.ProcessGroup.allreduce` per bucket on a group of 8 whose 7 other
    ranks' buckets are resident on the GPU, reduced in place into this rank's
    gradient with the divide fused, completion through the work's future; every
    work is waited for at the end of the step, as DDP's reducer does."""
    import datetime

    import torch.distributed as dist

    import fairring  # noqa: F401  (registers the backend, loads the extension)
    from fairring_amd import _fairring

    k, numel = args.k or 8, args.numel or 1_370_000_000
    slice_elems = args.slice_bytes // 4
    spans = ddp_buckets(numel, slice_elems, MiB // 4)
    if shared is not None:
        xs, own = shared       # `own` is overwritten: the group reduces in place
    else:
        xs = synth(torch, numel, k, "f32", 20240)
        own = torch.empty(numel, dtype=torch.float32, device="cuda:0")
    own.copy_(xs[0])
    torch.cuda.synchronize()
    o = _fairring.ProcessGroup.Options(
        max_memory_allocated_in_bytes=args.total_memory, max_padding_allocated_in_bytes=MiB,
        min_parallelism=2, is_high_priority_stream=True,
        timeout=datetime.timedelta(seconds=60), slice_size_in_bytes=args.slice_bytes)
    pg = _fairring.ProcessGroup(dist.HashStore(), 0, k, o)
    pg._set_fused_divide(True)
    own_views = [[own[lo:hi]] for lo, hi in spans]
    peer_views = [[x[lo:hi] for x in xs[1:]] for lo, hi in spans]

    def step():
        works = []
        for ov, pv in zip(own_views, peer_views):
            pg._set_simulated_peer_contributions(pv)
            works.append(pg.allreduce(ov))
        return works

    def finish(works):
        for w in works:
            w.wait()

    for _ in range(max(args.warmup, 1)):
        finish(step())
    pg._synchronize()
    torch.cuda.synchronize()
    pg._launch_records()        # drop what the warm-up left
    t0 = time.perf_counter()
    pg._profile_mark()
    pending = []
    for _ in range(args.steps):
        pending.append(step())
    pg._profile_mark()
    for works in pending:
        finish(works)
    pg._synchronize()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    recs = pg._launch_records()
    step_bytes = (k + 1) * numel * 4
    value = step_bytes * args.steps / elapsed / 1e9
    roof = roofline_from_records(recs, (k + 1) * 4,
                                 launch_elems(args, slice_elems, slice_elems, 4, k), SPAN_HOW)
    roof["kernel"] = "ksumKernel<F32Vec, SUM, K=%d>" % k
    # parity on a fresh copy of this rank's gradient (the timed steps reduced in place)
    own.copy_(xs[0])
    finish(step())
    pg._synchronize()
    torch.cuda.synchronize()
    checked = check_parity(oracle, np, torch, xs, own, numel, slice_elems, k, "f32", True)
    chain = xs[0].clone()
    for x in xs[1:]:
        chain.add_(x)
    chain.mul_(1.0 / k)
    same = torch.equal(own.view(torch.int32), chain.view(torch.int32))
    del chain
    if not same:
        raise SystemExit("parity FAILED against the at::add chain on the GPU (c5pg)")
    checked = "%s; every element equal to torch's at::add chain on the GPU" % checked
    layout = pg._layout()
    del pg
    cfg = {
        "workload": "DDP backward stream through _fairring.ProcessGroup.allreduce: %d fp32 "
                    "elements as %d buckets (first %d B, then %d B) released from the end of the "
                    "gradient to its start, group of %d (7 simulated peers resident on the GPU), "
                    "in place, fused x1/%d, every work waited for at the end of the step "
                    "(configs[4] through the drop-in surface)" % (
                        numel, len(spans), MiB, args.slice_bytes, k, k),
        "k": k, "numel": numel, "buckets": len(spans), "staging_total_bytes": args.total_memory,
        "layout": {"slot": layout[0], "slice": layout[1], "padding_slots": layout[2],
                   "staging_slots": layout[3]},
    }
    return value, elapsed, cfg, roof, checked, None, "f32"


def run_c5sep(args, np, torch, fa, oracle):
    """The bucket stream as DistributedDataParallel lays it out: every bucket an allocation of
    its own, and so is every peer's copy of it (48 buckets of 25 MiB, 8 contributions), one
    `_fairring.ProcessGroup.allreduce` per bucket, in place, divide fused, every work waited for
    at the end of the step. Nothing here is contiguous with anything else, so no two buckets
    can run as one operation."""
    import datetime

    import torch.distributed as dist

    import fairring  # noqa: F401  (registers the backend, loads the extension)
    from fairring_amd import _fairring

    k = args.k or 8
    buckets = 48
    n = args.slice_bytes // 4
    numel = args.numel or buckets * n
    buckets = max(1, numel // n)
    g = torch.Generator(device="cuda:0")
    g.manual_seed(515)
    # (In the default run this workload's tensors come from a memory pool of their own, see
    # main(): each is a segment from the driver, not a piece cut from a block that an earlier
    # workload left in torch's cache. Cut from 5 GB blocks the buckets start 25 MiB apart, 0
    # to 3 MiB past a multiple of a round of their allocation, and the stream runs 1.6 %
    # slower for it. The record says how many tensors start their allocation.)
    fresh = [torch.empty(n, device="cuda:0").normal_(0.0, 0.01, generator=g) for _ in range(buckets)]
    owns = [t.clone() for t in fresh]
    # (8 KiB of room behind every peer copy, for the second placement below; the allocator rounds
    # either size up to 26 MiB)
    room = [[torch.empty(n + 2048, device="cuda:0") for _ in range(k - 1)] for _ in range(buckets)]
    peers = [[buf[:n].normal_(0.0, 0.01, generator=g) for buf in row] for row in room]
    torch.cuda.synchronize()
    starts = {seg["address"] for seg in torch.cuda.memory_snapshot()}
    own_allocation = sum(t.data_ptr() in starts for row in [owns] + peers for t in row)
    o = _fairring.ProcessGroup.Options(
        max_memory_allocated_in_bytes=args.total_memory, max_padding_allocated_in_bytes=MiB,
        min_parallelism=2, is_high_priority_stream=True,
        timeout=datetime.timedelta(seconds=60), slice_size_in_bytes=args.slice_bytes)
    pg = _fairring.ProcessGroup(dist.HashStore(), 0, k, o)
    pg._set_fused_divide(True)
    own_lists = [[t] for t in owns]

    def step():
        works = []
        for ov, pv in zip(own_lists, peers):
            pg._set_simulated_peer_contributions(pv)
            works.append(pg.allreduce(ov))
        return works

    def finish(works):
        for w in works:
            w.wait()

    for _ in range(max(args.warmup, 1)):
        finish(step())
    pg._synchronize()
    torch.cuda.synchronize()
    pg._launch_records()
    steps = args.steps * 4          # a step is 11 GB: a few more of them for a steady figure
    t0 = time.perf_counter()
    pg._profile_mark()
    pending = [step() for _ in range(steps)]
    pg._profile_mark()
    for works in pending:
        finish(works)
    pg._synchronize()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    recs = pg._launch_records()
    value = (k + 1) * n * buckets * 4 * steps / elapsed / 1e9
    roof = roofline_from_records(recs, (k + 1) * 4, launch_elems(args, n, n, 4, k), SPAN_HOW)
    roof["kernel"] = "ksumKernel<F32Vec, SUM, K=%d>" % k
    # parity on fresh buckets (the timed steps reduced in place), three of them against the oracle
    for t, f in zip(owns, fresh):
        t.copy_(f)
    finish(step())
    pg._synchronize()
    torch.cuda.synchronize()
    checked = []
    for b in sorted({0, buckets // 2, buckets - 1}):
        host = [fresh[b].cpu().numpy()] + [p.cpu().numpy() for p in peers[b]]
        want = oracle.sum_f32(host, oracle.SCALE_MUL, 1.0 / k, threads=os.cpu_count() or 1)
        if not (owns[b].cpu().numpy().view(np.uint32) == want.view(np.uint32)).all():
            raise SystemExit("parity FAILED on bucket %d (c5sep)" % b)
        checked.append(b)
    # The same stream in the same allocations with peer copy j of every bucket starting j KiB
    # into its allocation instead of at its start: how much of this workload's rate is the
    # relative position of the nine tensors of a bucket within 4 KiB, which a caller that owns
    # the buffers the peers' contributions arrive in is free to choose.
    staggered = None
    if not args.numel:
        peers = [[buf[256 * (j + 1):256 * (j + 1) + n].normal_(0.0, 0.01, generator=g)
                  for j, buf in enumerate(row)] for row in room]
        torch.cuda.synchronize()
        for _ in range(max(args.warmup, 1)):
            finish(step())
        pg._synchronize()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        pending = [step() for _ in range(steps)]
        for works in pending:
            finish(works)
        pg._synchronize()
        torch.cuda.synchronize()
        staggered = (k + 1) * n * buckets * 4 * steps / (time.perf_counter() - t0) / 1e9
        for t, f in zip(owns, fresh):
            t.copy_(f)
        finish(step())
        pg._synchronize()
        torch.cuda.synchronize()
        for b in checked:
            host = [fresh[b].cpu().numpy()] + [p.cpu().numpy() for p in peers[b]]
            want = oracle.sum_f32(host, oracle.SCALE_MUL, 1.0 / k, threads=os.cpu_count() or 1)
            if not (owns[b].cpu().numpy().view(np.uint32) == want.view(np.uint32)).all():
                raise SystemExit("parity FAILED on bucket %d (c5sep, staggered peers)" % b)
    layout = pg._layout()
    del pg
    cfg = {
        "workload": "DDP-shaped bucket stream: %d buckets of %d B, each bucket and each of its %d "
                    "peer copies an allocation of its own, one _fairring.ProcessGroup.allreduce per "
                    "bucket, in place, fused x1/%d, every work waited for at the end of the step "
                    "(configs[4] with DistributedDataParallel's own bucket layout)" % (
                        buckets, args.slice_bytes, k - 1, k),
        "k": k, "numel": n * buckets, "buckets": buckets, "staging_total_bytes": args.total_memory,
        "tensors_at_the_start_of_their_allocation": "%d of %d" % (own_allocation, buckets * k),
        "layout": {"slot": layout[0], "slice": layout[1], "padding_slots": layout[2],
                   "staging_slots": layout[3]},
    }
    if staggered is not None:
        cfg["peer_copy_j_starting_j_KiB_into_its_allocation_GBps"] = round(staggered, 1)
    return value, elapsed / 4, cfg, roof, checked, None, "f32"


# One 25 MiB bucket of a transformer layer's gradients: two matrices, three vectors, a rest.
GATHER_SEGMENTS = [4194304, 2048, 2048, 2097152, 2048, 256000]


def run_gather(args, np, torch, fa, oracle, shared=None):
    """The bucket stream of DistributedDataParallel with gradient_as_bucket_view=False (its
    default): every bucket an allocation of its own (48 of 25 MiB, as in c5sep), this rank's
    contribution still in the gradient tensors autograd left it in (six per bucket, tensors of
    their own), one `_fairring.ProcessGroup._allreduce_from_grads` per bucket, which reads the
    gradients themselves and writes the bucket once. Beside it the same stream the way the
    reducer does it: every gradient copied into its bucket first (one copy kernel per tensor),
    then `allreduce` on the bucket in place."""
    import datetime

    import torch.distributed as dist

    import fairring  # noqa: F401  (registers the backend, loads the extension)
    from fairring_amd import _fairring

    k = args.k or 8
    n = args.slice_bytes // 4
    buckets = max(1, (args.numel or 48 * n) // n)
    seg_lens = [ln for ln in GATHER_SEGMENTS]
    if sum(seg_lens) != n:                      # another slice size: one tensor takes the rest
        seg_lens = [min(ln, n) for ln in GATHER_SEGMENTS[:1]] + [max(0, n - min(GATHER_SEGMENTS[0], n))]
        seg_lens = [ln for ln in seg_lens if ln > 0]
    g = torch.Generator(device="cuda:0")
    g.manual_seed(616)

    def fresh(numel):
        return torch.empty(numel, device="cuda:0").normal_(0.0, 0.01, generator=g)

    grads = [[fresh(ln) for ln in seg_lens] for _ in range(buckets)]
    bucket_of = [torch.empty(n, device="cuda:0") for _ in range(buckets)]
    peers = [[fresh(n) for _ in range(k - 1)] for _ in range(buckets)]
    torch.cuda.synchronize()
    o = _fairring.ProcessGroup.Options(
        max_memory_allocated_in_bytes=args.total_memory, max_padding_allocated_in_bytes=MiB,
        min_parallelism=2, is_high_priority_stream=True,
        timeout=datetime.timedelta(seconds=60), slice_size_in_bytes=args.slice_bytes)
    pg = _fairring.ProcessGroup(dist.HashStore(), 0, k, o)
    pg._set_fused_divide(True)

    def step():
        works = []
        for b, gr, pv in zip(bucket_of, grads, peers):
            pg._set_simulated_peer_contributions(pv)
            works.append(pg._allreduce_from_grads(b, gr))
        return works

    def two_pass():
        works = []
        for b, gr, pv in zip(bucket_of, grads, peers):
            at = 0
            for t in gr:
                b[at:at + t.numel()].copy_(t)
                at += t.numel()
            pg._set_simulated_peer_contributions(pv)
            works.append(pg.allreduce([b]))
        return works

    def finish(works):
        for w in works:
            w.wait()

    def run(fn, steps, marks):
        for _ in range(max(args.warmup, 1)):
            finish(fn())
        pg._synchronize()
        torch.cuda.synchronize()
        pg._launch_records()
        t0 = time.perf_counter()
        if marks:
            pg._profile_mark()
        pending = [fn() for _ in range(steps)]
        if marks:
            pg._profile_mark()
        for works in pending:
            finish(works)
        pg._synchronize()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    steps = args.steps * 4          # a step is 11 GB: a few more of them for a steady figure
    step_bytes = (k + 1) * n * buckets * 4
    elapsed = run(step, steps, True)
    recs = pg._launch_records()
    value = step_bytes * steps / elapsed / 1e9
    roof = roofline_from_records(recs, (k + 1) * 4, launch_elems(args, n, n, 4, k), SPAN_HOW)
    roof["kernel"] = ("ksumKernel<F32Vec, SUM, K=%d> for launches within one gradient, "
                      "ksumSegmentedKernel<F32Vec, K=%d, x1/%d> for those that hold several" % (k, k, k))
    # parity of three buckets against the oracle, and of every bucket against copy + allreduce
    got = [b.clone() for b in bucket_of]
    checked = []
    for i in sorted({0, buckets // 2, buckets - 1}):
        own = torch.cat(grads[i]).cpu().numpy()
        host = [own] + [p.cpu().numpy() for p in peers[i]]
        want = oracle.sum_f32(host, oracle.SCALE_MUL, 1.0 / k, threads=os.cpu_count() or 1)
        if not (got[i].cpu().numpy().view(np.uint32) == want.view(np.uint32)).all():
            raise SystemExit("parity FAILED on bucket %d (gather)" % i)
        checked.append(i)
    two = step_bytes * steps / run(two_pass, steps, False) / 1e9
    for i, (a, b) in enumerate(zip(got, bucket_of)):
        if not torch.equal(a.view(torch.int32), b.view(torch.int32)):
            raise SystemExit("parity FAILED: gathered differs from copy + allreduce (bucket %d)" % i)
    # The same buckets under torch's bf16 compression hook: 7 peers' bf16 tensors per bucket,
    # the own fp32 contribution read from the gradients (frg_allreduce_compressed_gathered),
    # against copy-then-compressed-allreduce; 4 + 7 x 2 + 4 = 22 algorithmic bytes per element.
    wire_peers = [[p.to(torch.bfloat16) for p in pv] for pv in peers]
    del peers
    torch.cuda.synchronize()

    def hook_step():
        works = []
        for b, gr, pv in zip(bucket_of, grads, wire_peers):
            pg._set_simulated_peer_contributions(pv)
            works.append(pg._allreduce_compressed(b, torch.bfloat16, gr))
        return works

    def hook_two_pass():
        works = []
        for b, gr, pv in zip(bucket_of, grads, wire_peers):
            at = 0
            for t in gr:
                b[at:at + t.numel()].copy_(t)
                at += t.numel()
            pg._set_simulated_peer_contributions(pv)
            works.append(pg._allreduce_compressed(b, torch.bfloat16))
        return works

    hook_bytes = (4 + 2 * (k - 1) + 4) * n * buckets
    hook_one = hook_bytes * steps / run(hook_step, steps, False) / 1e9
    got_hook = [b.clone() for b in bucket_of]
    hook_two = hook_bytes * steps / run(hook_two_pass, steps, False) / 1e9
    for i, (a, b) in enumerate(zip(got_hook, bucket_of)):
        if not torch.equal(a.view(torch.int32), b.view(torch.int32)):
            raise SystemExit("parity FAILED: compressed from gradients differs from copy + "
                             "compressed allreduce (bucket %d)" % i)
    own0 = torch.cat(grads[0]).cpu().numpy()
    want0 = oracle.compressed_sum(
        [own0] + [p.view(torch.int16).cpu().numpy().view(np.uint16) for p in wire_peers[0]], 0,
        "bf16", oracle.SCALE_MUL, float(np.float32(1) / np.float32(k)), threads=os.cpu_count() or 1)
    if not (got_hook[0].cpu().numpy().view(np.uint32) == want0.view(np.uint32)).all():
        raise SystemExit("parity FAILED on bucket 0 (compressed from gradients)")
    layout = pg._layout()
    del pg
    cfg = {
        "workload": "DDP-shaped bucket stream with this rank's contribution read from its gradient "
                    "tensors: %d buckets of %d B, each bucket, each of its %d peer copies and each "
                    "of its %d gradient tensors (%s elements) an allocation of its own, one "
                    "_fairring.ProcessGroup._allreduce_from_grads per bucket, fused x1/%d; the copy "
                    "of every gradient into its bucket (8 bytes per element) is not made" % (
                        buckets, n * 4, k - 1, len(seg_lens), "/".join(str(v) for v in seg_lens),
                        k),
        "k": k, "numel": n * buckets, "buckets": buckets, "tensors": buckets * len(seg_lens),
        "copy_then_allreduce_GBps": round(two, 1),
        "copy_then_allreduce_note": "same algorithmic bytes over the time of copying every "
                                    "gradient into its bucket (torch's copy kernels) and "
                                    "ProcessGroup.allreduce on the bucket in place; results equal "
                                    "bit for bit",
        "bf16_hook_from_grads_GBps": round(hook_one, 1),
        "bf16_hook_copy_then_allreduce_GBps": round(hook_two, 1),
        "bf16_hook_note": "the same buckets with torch's bf16 compression hook folded in (7 bf16 "
                          "peers per bucket, 22 algorithmic bytes per element): own fp32 "
                          "contribution read from the gradients, against copying them into the "
                          "bucket first; results equal bit for bit, bucket 0 against the oracle",
        "staging_total_bytes": args.total_memory,
        "layout": {"slot": layout[0], "slice": layout[1], "padding_slots": layout[2],
                   "staging_slots": layout[3]},
    }
    return value, elapsed / 4, cfg, roof, checked, None, "f32"


def run_hook(args, np, torch, fa, oracle):
    """The reduction with torch's bf16 compression hook folded in: this rank's
    fp32 gradient is compressed in registers, K - 1 peers' bf16 tensors are read,
    the result is decompressed in place into the fp32 gradient. 4 + 2 (K - 1) + 4
    algorithmic bytes per element."""
    k, numel = args.k or 8, args.numel or 1_370_000_000
    slice_elems = args.slice_bytes // 2          # sliced as the bf16 tensor the hook hands over
    n_slices = (numel + slice_elems - 1) // slice_elems
    raw = 0
    dev = fa.DeviceFairring(0, max_memory_allocated_in_bytes=args.total_memory,
                            slice_size_in_bytes=args.slice_bytes,
                            num_reduce_streams=args.streams,
                            max_launch_bytes=args.launch_bytes)
    peers = synth(torch, numel, k, "bf16", 20240)
    bucket = synth(torch, numel, 1, "f32", 777)[0]
    contribs = list(peers)
    contribs[raw] = bucket
    del peers
    torch.cuda.synchronize()
    inv = float(np.float32(1) / np.float32(k))

    def step(d):
        return d.allreduce_compressed(bucket, contribs, raw, scale_mode=fa.SCALE_MUL, scale=inv)

    elapsed, recs = timed(torch, dev, args.steps, args.warmup, step)
    bytes_per_elem = 4 + 2 * (k - 1) + 4
    value = bytes_per_elem * numel * args.steps / elapsed / 1e9
    # the library's default for the compressed reduction (layout.h::defaultCompressedLaunchBytes):
    # whole rounds of 2 MiB of wire nearest to 80 MB per launch; a bucket is one launch
    if k <= 8 and numel * 2 < 100 * MiB:
        default_lb = 16 * MiB
    else:
        default_lb = max(1, -(-(2 * 80 * MiB // bytes_per_elem) // (2 * MiB))) * 2 * MiB
    roof = roofline_from_records(recs, bytes_per_elem,
                                 launch_elems(args, numel, slice_elems, 2,
                                              compressed_default=default_lb), SPAN_HOW)
    roof["kernel"] = "compressedKernel<Bf16Vec, out fp32>, K=%d" % k
    # parity on a fresh bucket (the timed steps reduced in place)
    fresh = synth(torch, numel, 1, "f32", 777)[0]
    bucket.copy_(fresh)
    step(dev).wait()
    checked = []
    for idx in sorted({0, n_slices // 2, n_slices - 1}):
        lo, hi = idx * slice_elems, min(numel, (idx + 1) * slice_elems)
        host = [to_host(np, torch, c[lo:hi]) for c in contribs]
        host[raw] = fresh[lo:hi].cpu().numpy()
        want = oracle.compressed_sum(host, raw, "bf16", oracle.SCALE_MUL, inv,
                                     threads=os.cpu_count() or 1)
        got = bucket[lo:hi].cpu().numpy()
        if not (got.view(np.uint32) == want.view(np.uint32)).all():
            raise SystemExit("parity FAILED on slice %d" % idx)
        checked.append(idx)
    layout = dev.layout
    dev.close()
    cfg = {
        "workload": "bf16 compression hook folded into the reduction: own fp32 gradient of %d "
                    "elements + %d peers' bf16 tensors, %d slices of %d B (bf16), x1/%d on the own "
                    "term, result decompressed in place into the fp32 gradient" % (
                        numel, k - 1, n_slices, args.slice_bytes, k),
        "k": k, "numel": numel, "slice_bytes": args.slice_bytes,
        "staging_total_bytes": args.total_memory, "layout": layout,
        "reduce_streams": args.streams or "default",
        "launch_bytes_per_contribution": args.launch_bytes or "default",
    }
    return value, elapsed, cfg, roof, checked, None, "bf16"


def run_placement(args, torch, fa):
    """The 8-way fp32 reduction of a 400 M-element gradient at several placements of its nine
    buffers in one process: before each placement something else takes memory first, of
    another size each time, so the buffers land elsewhere in HBM (everything stays allocated
    until the end). Prints its own JSON line
    with the rate at each placement (host clock over `--steps` passes after one warm-up
    pass). Under `rocprofv3 --pmc` (dispatches serialised) the per-dispatch counter records
    of each placement are what shows whether placements differ in how they load the memory
    channels."""
    import time
    k, n = args.k or 8, args.numel or 400_000_000
    dev = fa.DeviceFairring(0, slice_size_in_bytes=args.slice_bytes,
                            max_memory_allocated_in_bytes=args.total_memory)
    g = torch.Generator(device="cuda:0")
    spacers, report, held = [], [], []
    for r in range(6):
        g.manual_seed(100 + r)
        spacers.append(torch.empty((r * 777 + 300) << 20, dtype=torch.uint8, device="cuda:0"))
        xs = [torch.empty(n, device="cuda:0").normal_(0, 0.01, generator=g) for _ in range(k)]
        out = torch.empty(n, device="cuda:0")
        torch.cuda.synchronize()
        dev.allreduce(out, xs, scale_mode=fa.SCALE_MUL, scale=1.0 / k).wait()
        dev.synchronize()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        w = None
        for _ in range(args.steps):
            w = dev.allreduce(out, xs, scale_mode=fa.SCALE_MUL, scale=1.0 / k)
        w.wait()
        dev.synchronize()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        report.append({"out": "%#x" % out.data_ptr(), "first_contribution": "%#x" % xs[0].data_ptr(),
                       "GBps": round((k + 1) * 4 * n * args.steps / dt / 1e9, 1)})
        # nothing is freed between placements (14 GB each): memory that has just gone back to
        # the driver slows down whatever runs next, which is not what is measured here
        held.append((xs, out))
    dev.close()
    rates = sorted(p["GBps"] for p in report)
    print(json.dumps({"metric": "reduce GB/s (bytes read+written), 8-way fp32, by placement of the "
                                "buffers", "unit": "GB/s", "value": rates[len(rates) // 2],
                      "min": rates[0], "max": rates[-1], "n_gpus": 1, "steps": args.steps,
                      "k": k, "numel": n, "placements": report}))


def run_small_ops(args, torch, fa):
    """Per-operation cost at bucket sizes where the kernel is short (a DDP step's
    first 1 MiB bucket and its small ones): what the caller's thread pays per
    call, call -> wait -> device idle, and the sustained back-to-back rate,
    through the ctypes mirror of the ABI and, when the torch extension is built,
    through the process group. Prints its own JSON line (operations per second)."""
    import datetime
    import time
    k = args.k or 8
    sizes = [1024, 262144]
    reps, burst = 200, max(args.steps, 1) * 100

    def measure(submit, wait_last):
        out = {}
        for numel in sizes:
            call = submit(numel)
            wait_last(call())
            torch.cuda.synchronize()
            lat = []
            for _ in range(reps):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                wait_last(call())
                torch.cuda.synchronize()
                lat.append(time.perf_counter() - t0)
            lat.sort()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(burst):
                w = call()
            t1 = time.perf_counter()
            wait_last(w)
            torch.cuda.synchronize()
            t2 = time.perf_counter()
            out[str(numel)] = {"latency_us_median": round(lat[reps // 2] * 1e6, 1),
                               "latency_us_p90": round(lat[reps * 9 // 10] * 1e6, 1),
                               "caller_us_per_op": round((t1 - t0) / burst * 1e6, 1),
                               "sustained_us_per_op": round((t2 - t0) / burst * 1e6, 1)}
        return out

    dev = fa.DeviceFairring(0)

    # Operations on distinct tensors, like the buckets of a gradient: the pipeline
    # lets them overlap. (Operations that share a tensor are ordered with an event
    # between the streams; "in_place_chain" below is that case.)
    import itertools

    def submit_abi(numel):
        xs = [torch.zeros(numel, device="cuda:0") for _ in range(k)]
        outs = itertools.cycle([torch.empty(numel, device="cuda:0") for _ in range(4)])
        return lambda: dev.allreduce(next(outs), xs)

    report = {"abi_ctypes": measure(submit_abi, lambda w: w.wait())}
    dev.close()
    try:
        import torch.distributed as dist

        import fairring  # noqa: F401  (registers the backend, loads the extension)
        from fairring_amd import _fairring
    except ImportError:
        _fairring = None
    if _fairring is not None:
        o = _fairring.ProcessGroup.Options(
            max_memory_allocated_in_bytes=args.total_memory,
            max_padding_allocated_in_bytes=MiB, min_parallelism=2, is_high_priority_stream=True,
            timeout=datetime.timedelta(seconds=60), slice_size_in_bytes=args.slice_bytes)
        pg = _fairring.ProcessGroup(dist.HashStore(), 0, k, o)

        def submit_pg(numel, distinct=4):
            owns = itertools.cycle([[torch.zeros(numel, device="cuda:0")]
                                    for _ in range(distinct)])
            pg._set_simulated_peer_contributions(
                [torch.zeros(numel, device="cuda:0") for _ in range(k - 1)])
            return lambda: pg.allreduce(next(owns))

        report["process_group"] = measure(submit_pg, lambda w: w.wait())
        report["process_group_in_place_chain"] = measure(lambda n: submit_pg(n, 1),
                                                         lambda w: w.wait())
    # the one-launch entry point on the caller's stream: eager, and the same loop captured
    # once into a HIP graph and replayed (it allocates nothing and records no event)
    nb = 64
    xs = [[torch.zeros(sizes[1], device="cuda:0") for _ in range(k)] for _ in range(nb)]
    outs = [torch.empty(sizes[1], device="cuda:0") for _ in range(nb)]

    def loop():
        for o, c in zip(outs, xs):
            fa.reduce_slice(o, c, scale_mode=fa.SCALE_MUL, scale=1.0 / k)

    loop()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        loop()
    rounds = max(burst // nb, 1)
    direct = {}
    for name, fn in (("eager", loop), ("graph_replay", graph.replay)):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(rounds):
            fn()
        torch.cuda.synchronize()
        direct[name + "_us_per_launch"] = round((time.perf_counter() - t0) / (rounds * nb) * 1e6, 2)
    report["reduce_slice_%d_elements" % sizes[1]] = direct
    best = report.get("process_group", report["abi_ctypes"])[str(sizes[0])]
    print(json.dumps({
        "metric": "small allreduce operations per second, %d-way fp32, back to back" % k,
        "value": round(1e6 / best["sustained_us_per_op"], 1), "unit": "operations/s",
        "n_gpus": 1, "steps": burst, "warmup": 1, "higher_is_better": True,
        "dtype": "f32", "data": "synthetic: zeros", "vs_baseline": None,
        "config": {"workload": "smallops", "k": k, "elements": sizes}, "detail": report}))


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path, run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import fairring_amd as fa
    import oracle
    from fairring_amd import _capi

    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")
    _capi.lib()  # fail now if the HIP library is missing
    if args.blocks_per_cu:
        _capi.lib().frg_set_tuning(args.blocks_per_cu)

    if args.workload == "smallops":
        run_small_ops(args, torch, fa)
        return
    if args.workload == "placement":
        run_placement(args, torch, fa)
        return

    keep = []
    result = measure(args, args.workload, np, torch, fa, oracle, keep=keep)
    failed = []
    if args.workload == "c2" and not args.no_extra_configs and not (
            args.k or args.numel or args.launch_bytes or args.streams or args.blocks_per_cu):
        # The other workloads, briefly, for the record: same code paths as when
        # they are run on their own, fewer steps, no CPU baseline.
        shared = tuple(keep) if keep else None
        extra = {}
        pools = []
        for name in [x for x in args.extras.split(",") if x]:
            sub = argparse.Namespace(**vars(args))
            sub.workload, sub.no_cpu_baseline = name, True
            # (c3 moves 1.7 GB over the host link per step, the others 11 to 49 GB
            # within HBM)
            # As many steps and warm-up steps as the headline, up to 50 after 100.
            sub.steps = min(args.steps, 3 if name == "c3" else 50)
            sub.warmup = min(args.warmup, 2 if name == "c3" else 100)
            if name in ("c5sep", "gather"):
                sub.warmup = min(args.warmup * 4, 400)     # a step of them is 11 GB, not 49
            if name in ("gather", "c5sep", "c4"):
                shared = None
                keep.clear()       # the fp32 inputs go before other ones are made
            # (Memory is not handed back to the driver between workloads: what is allocated
            # right after tens of GB were released is slower for it. The bf16 workload ran at
            # 6,230 GB/s on such memory against 6,618 on blocks torch had kept and 6,659 in a
            # fresh process; a staging pool allocated then took host copies at half the link's
            # rate, 27 against 54 GB/s, until 3 s had passed.)
            try:
                if name in ("c5", "c5pg"):
                    r = measure(sub, name, np, torch, fa, oracle, shared=shared)
                else:
                    # Tensors of its own, from the driver, as in a run of its own: a memory
                    # pool per workload, kept until the process ends (see above: memory must
                    # not go back to the driver in between).
                    pools.append(torch.cuda.MemPool())
                    with torch.cuda.use_mem_pool(pools[-1]):
                        r = measure(sub, name, np, torch, fa, oracle)
                # compact: the whole record stays one line of a few KB
                roof = {key: r["roofline"][key] for key in (
                    "bound", "achieved", "peak", "nominal", "unit", "frac", "traffic",
                    "launch_bytes", "avg_launch_us", "concurrency", "kernel", "hbm")
                    if key in r["roofline"]}
                extra[name] = {"metric": r["metric"], "value": r["value"], "unit": r["unit"],
                               "steps": r["steps"], "ms_per_step": r["ms_per_step"],
                               "dtype": r["dtype"], "pct_of_hbm_peak": r["pct_of_hbm_peak"],
                               "parity": r["parity"].split(";")[0], "roofline": roof}
                for key in ("host_link_GBps", "copy_then_allreduce_GBps",
                            "bf16_hook_from_grads_GBps", "bf16_hook_copy_then_allreduce_GBps",
                            "tensors_at_the_start_of_their_allocation",
                            "peer_copy_j_starting_j_KiB_into_its_allocation_GBps"):
                    if key in r["config"]:
                        extra[name][key] = r["config"][key]
            except (SystemExit, Exception) as e:  # noqa: BLE001  (reported, and the run fails)
                extra[name] = {"error": "%s: %s" % (type(e).__name__, e)}
                failed.append(name)
        result["configs"] = extra
    del keep[:]
    if callable(result.get("cpu_baseline")):
        result["cpu_baseline"] = result["cpu_baseline"]()
    print(json.dumps(result))
    if failed:
        sys.exit("workloads that failed: %s" % ", ".join(failed))


def measure(args, workload, np, torch, fa, oracle, keep=None, shared=None):
    """Runs one workload and returns its result line as a dict."""
    if workload in ("c2", "copy"):
        value, elapsed, cfg, roof, checked, base, dtype = run_resident(
            args, np, torch, fa, oracle, "f32", keep=keep if workload == "c2" else None)
    elif workload == "c4":
        value, elapsed, cfg, roof, checked, base, dtype = run_resident(args, np, torch, fa,
                                                                       oracle, "bf16")
    elif workload == "c3":
        value, elapsed, cfg, roof, checked, base, dtype = run_c3(args, np, torch, fa, oracle)
    elif workload == "hook":
        value, elapsed, cfg, roof, checked, base, dtype = run_hook(args, np, torch, fa, oracle)
    elif workload == "c5pg":
        value, elapsed, cfg, roof, checked, base, dtype = run_c5pg(args, np, torch, fa, oracle,
                                                                   shared=shared)
    elif workload == "c5sep":
        value, elapsed, cfg, roof, checked, base, dtype = run_c5sep(args, np, torch, fa, oracle)
    elif workload == "gather":
        value, elapsed, cfg, roof, checked, base, dtype = run_gather(args, np, torch, fa, oracle,
                                                                     shared=shared)
    else:
        value, elapsed, cfg, roof, checked, base, dtype = run_c5(args, np, torch, fa, oracle,
                                                                 shared=shared)

    # HBM bytes per launch as measured with rocprofv3 --pmc (two counter runs,
    # scaled by a copy of known size) in an earlier run of the same command: a
    # constant read from the summary named in traffic_source, not measured now.
    traffic_file = {"c2": "ksum_f32_k8_c2_hbm_traffic.md",
                    "hook": "compressed_bf16_k8_hook_hbm_traffic.md"}.get(workload)
    if (traffic_file and args.slice_bytes == 25 * MiB and not args.k and not args.numel
            and not args.launch_bytes):
        tpath = os.path.join(ROOT, "profiles", traffic_file)
        if os.path.exists(tpath):
            import re
            text = open(tpath).read()
            m = re.search(r"traffic = [\d,]+ KiB = ([\d,]+) B per launch", text)
            at = re.search(r"[Mm]easured at commit ([0-9a-f]{7,40})", text)
            if m:
                roof["traffic"] = int(m.group(1).replace(",", ""))
                roof["traffic_source"] = ("profiles/%s (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                                          "of an earlier run of this command%s; not measured in "
                                          "this run)" % (traffic_file,
                                                         ", at commit %s" % at.group(1) if at else ""))

    metric = {
        "c2": "reduce GB/s (bytes read+written), 8-way fp32, 25 MiB slices",
        "c4": "reduce GB/s (bytes read+written), 8-way bf16, 25 MiB slices",
        "c3": "reduce GB/s (bytes read+written at HBM level), 64-way fp32 host-staged, one slice",
        "c5": "reduce GB/s (bytes read+written), 8-way fp32 DDP bucket stream",
        "c5pg": "reduce GB/s (bytes read+written), 8-way fp32 DDP bucket stream through "
                "ProcessGroup.allreduce",
        "c5sep": "reduce GB/s (bytes read+written), 8-way fp32 bucket stream, every bucket and "
                 "contribution its own allocation, through ProcessGroup.allreduce",
        "gather": "reduce GB/s (bytes read+written), 8-way fp32 bucket stream, own contribution "
                  "read from the gradient tensors",
        "copy": "copy GB/s (bytes read+written), 25 MiB slices",
        "hook": "reduce GB/s (bytes read+written), 8-way with the bf16 compression hook folded in",
    }[workload]
    result = {
        "metric": metric,
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype,
        "data": "synthetic: N(0, sigma=0.01) per contribution from fixed seeds, resident before "
                "the timed region",
        "config": cfg,
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "parity": "bit-exact vs CPU oracle on slices %s" % checked,
        "roofline": roof,
    }
    if base is not None:
        result["cpu_baseline"] = base
    return result


if __name__ == "__main__":
    main()
