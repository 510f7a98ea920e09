"""Host-side mirror of the reference's per-GPU object on top of the C ABI.

``DeviceFairring`` plays the role of fairring/device.h:22-117 for one MI355X:
it owns a pipeline context (streams, staging pool, command thread) and turns
``allreduce`` calls on torch tensors into asynchronous slice reductions.
PyTorch is used here for device memory and the current stream only.
"""
import ctypes
import os
import sys

from . import _capi
from ._capi import (BF16, F16, F32, F64, I8, I32, I64, MAX, SCALE_DIV, SCALE_MUL,
                    SCALE_NONE, SCALE_PRE_DIV, SCALE_PRE_MUL, SUM, U8, FairringError)

MiB = 1024 * 1024


def options_from_env(environ=None, stderr=None):
    """Staging options from the environment, as fairring/__init__.py:17-34 reads
    them, plus the FAIRRING_SLICE_SIZE of README.md:62."""
    env = os.environ if environ is None else environ
    err = sys.stderr if stderr is None else stderr
    opts = {}
    try:
        opts["max_memory_allocated_in_bytes"] = int(env["FAIRRING_TOTAL_MEMORY"])
    except KeyError:
        err.write(
            "The Fairring process group will allocate up to 50 MiB of staging memory "
            "on each GPU. This can be tuned by setting the FAIRRING_TOTAL_MEMORY "
            "environment variable (to an amount of bytes).\n")
        opts["max_memory_allocated_in_bytes"] = 50 * MiB
    try:
        opts["max_padding_allocated_in_bytes"] = int(env["FAIRRING_PADDING_MEMORY"])
    except KeyError:
        opts["max_padding_allocated_in_bytes"] = MiB
    try:
        opts["min_parallelism"] = int(env["FAIRRING_PARALLELISM"])
    except KeyError:
        opts["min_parallelism"] = 16
    if "FAIRRING_SLICE_SIZE" in env:
        opts["slice_size_in_bytes"] = int(env["FAIRRING_SLICE_SIZE"])
    return opts


def compute_layout(max_memory, max_padding, min_parallelism, num_machines, devices_per_machine):
    out = _capi.Layout()
    _capi.check(_capi.lib().frg_compute_layout(max_memory, max_padding, min_parallelism,
                                               num_machines, devices_per_machine,
                                               ctypes.byref(out)))
    return dict(slot=out.slot_size_in_bytes, slice=out.slice_size_in_bytes,
                padding_slots=out.num_padding_slots, staging_slots=out.num_staging_slots)


def plan_launches(k, numel, element_size, first_contribution_address=0,
                  out_offset_in_allocation=0, align_short_operations=False, num_cus=256):
    """The launches the pipeline cuts an operation into by default:
    [(elements, blocks per CU), ...] in order (frg_plan_launches)."""
    cap = 1 << 16
    elems = (ctypes.c_int64 * cap)()
    bpc = (ctypes.c_int32 * cap)()
    n = ctypes.c_int()
    _capi.check(_capi.lib().frg_plan_launches(k, numel, element_size, first_contribution_address,
                                              out_offset_in_allocation,
                                              1 if align_short_operations else 0, num_cus, elems,
                                              bpc, cap, ctypes.byref(n)))
    return [(elems[i], bpc[i]) for i in range(min(n.value, cap))]


def _dtype_code(t):
    import torch
    codes = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16, torch.float64: F64,
             torch.int32: I32, torch.int64: I64, torch.uint8: U8, torch.int8: I8}
    try:
        return codes[t.dtype]
    except KeyError:
        raise FairringError(_capi.ERR_UNSUPPORTED, "unsupported dtype %s" % t.dtype)


def is_non_overlapping_and_dense(t):
    """True when the tensor's elements fill one contiguous range of memory in
    some dimension order (what viewAsFlat requires, fairring/utils.h:353-361)."""
    dims = sorted((st, sz) for sz, st in zip(t.shape, t.stride()) if sz != 1)
    expect = 1
    for st, sz in dims:
        if sz == 0:
            return True
        if st != expect:
            return False
        expect *= sz
    return True


def _check_dense(t, what, device=True):
    import torch
    if t.layout != torch.strided:
        raise FairringError(_capi.ERR_INVALID, "%s must be strided" % what)
    if device and not t.is_cuda:
        raise FairringError(_capi.ERR_INVALID, "%s must be a GPU tensor" % what)
    if not is_non_overlapping_and_dense(t):
        raise FairringError(_capi.ERR_INVALID, "%s must be non-overlapping and dense" % what)


def reduce_slice(out, contribs, op=SUM, scale_mode=SCALE_NONE, scale=1.0, carry=False,
                 stream=None):
    """One reduction launch (doReduction, fairring/device.cc:108-131) on torch
    GPU tensors, on `stream` (default: torch's current stream)."""
    import torch
    stream = torch.cuda.current_stream(out.device) if stream is None else stream
    tab = _capi.ptr_table([c.data_ptr() for c in contribs])
    for c in contribs:
        if c.numel() != out.numel() or c.dtype != out.dtype:
            raise FairringError(_capi.ERR_INVALID, "contribution shape/dtype mismatch")
    _capi.check(_capi.lib().frg_reduce_slice(
        out.data_ptr(), tab, len(contribs), out.numel(), _dtype_code(out), op, scale_mode,
        scale, 1 if carry else 0, stream.cuda_stream))


def reduce_slice_static(out, contribs, op=SUM, scale_mode=SCALE_NONE, scale=1.0, stream=None):
    """reduce_slice for any number of contributions without any allocation
    (frg_reduce_slice_static): chains of more than 64 park their partial result
    in the library's static device array."""
    import torch
    stream = torch.cuda.current_stream(out.device) if stream is None else stream
    for c in contribs:
        if c.numel() != out.numel() or c.dtype != out.dtype:
            raise FairringError(_capi.ERR_INVALID, "contribution shape/dtype mismatch")
    tab = _capi.ptr_table([c.data_ptr() for c in contribs])
    _capi.check(_capi.lib().frg_reduce_slice_static(
        out.data_ptr(), tab, len(contribs), out.numel(), _dtype_code(out), op, scale_mode, scale,
        stream.cuda_stream))


def reduce_pieces(pieces, op=SUM, scale_mode=SCALE_NONE, scale=1.0, stream=None):
    """Several reductions of one kind as one call (frg_reduce_pieces): `pieces`
    is a list of (out, [contributions]) with the same number of contributions
    and dtype throughout; small tensors share launches."""
    import torch
    if not pieces:
        return
    out0, c0 = pieces[0]
    stream = torch.cuda.current_stream(out0.device) if stream is None else stream
    k = len(c0)
    arr = (_capi.Piece * len(pieces))()
    keep = []
    for i, (out, contribs) in enumerate(pieces):
        if len(contribs) != k or out.dtype != out0.dtype:
            raise FairringError(_capi.ERR_INVALID, "pieces differ in kind")
        for c in contribs:
            if c.numel() != out.numel() or c.dtype != out.dtype:
                raise FairringError(_capi.ERR_INVALID, "contribution shape/dtype mismatch")
        tab = _capi.ptr_table([c.data_ptr() for c in contribs])
        keep.append(tab)
        arr[i].out = out.data_ptr()
        arr[i].contribs = ctypes.cast(tab, ctypes.POINTER(ctypes.c_void_p))
        arr[i].numel = out.numel()
    _capi.check(_capi.lib().frg_reduce_pieces(arr, len(pieces), k, _dtype_code(out0), op,
                                              scale_mode, scale, stream.cuda_stream))


def _check_compressed(out, contribs, raw_index):
    """Shapes and types of the reduction with compression folded in; returns
    the wire dtype code."""
    import torch
    if not -1 <= raw_index < len(contribs):
        raise FairringError(_capi.ERR_INVALID, "raw_index out of range")
    wire = None
    for k, c in enumerate(contribs):
        if c.numel() != out.numel():
            raise FairringError(_capi.ERR_INVALID, "contribution shape mismatch")
        if k == raw_index:
            if c.dtype != torch.float32:
                raise FairringError(_capi.ERR_INVALID, "the raw contribution must be float32")
        elif wire is None:
            wire = c.dtype
        elif c.dtype != wire:
            raise FairringError(_capi.ERR_INVALID, "peers' contributions differ in dtype")
    if wire is None:
        wire = out.dtype if out.dtype != torch.float32 else torch.bfloat16
    if wire not in (torch.bfloat16, torch.float16):
        raise FairringError(_capi.ERR_UNSUPPORTED, "the wire type must be bfloat16 or float16")
    if out.dtype not in (torch.float32, wire):
        raise FairringError(_capi.ERR_UNSUPPORTED, "the output must be float32 or of the wire type")
    return BF16 if wire == torch.bfloat16 else F16


def reduce_slice_compressed(out, contribs, raw_index=-1, scale_mode=SCALE_NONE, scale=1.0,
                            wire_dtype=None, stream=None):
    """One launch of the reduction with torch's bf16 / fp16 compression hooks
    folded in (torch:distributed/algorithms/ddp_comm_hooks/default_hooks.py:57-93):
    contribs[raw_index] is this rank's float32 bucket, cast to the wire type and
    scaled there in registers; the others are peers' tensors in the wire type;
    `out` is of the wire type, or float32 to receive the result widened (it may
    be the raw bucket itself). `wire_dtype` is only needed when there is no
    peer tensor to take it from."""
    import torch
    stream = torch.cuda.current_stream(out.device) if stream is None else stream
    wire = _check_compressed(out, contribs, raw_index)
    if wire_dtype is not None:
        wire = BF16 if wire_dtype == torch.bfloat16 else F16
    tab = _capi.ptr_table([c.data_ptr() for c in contribs])
    _capi.check(_capi.lib().frg_reduce_slice_compressed(
        out.data_ptr(), _dtype_code(out), tab, len(contribs), raw_index, out.numel(), wire,
        scale_mode, scale, stream.cuda_stream))


def set_wait_timeout(seconds):
    """Process-wide limit of Work.wait() in seconds; 0 = none. A wait that gives
    up raises FairringError (ERR_NOT_READY) with a report of where the pipeline
    stands, and can be repeated."""
    _capi.check(_capi.lib().frg_set_wait_timeout(float(seconds)))


class Work:
    """Handle on a submitted operation (WorkFairring, process_group.cc:35-75)."""

    def __init__(self, handle, keepalive):
        self._h = handle
        self._keep = keepalive

    def is_completed(self):
        return _capi.lib().frg_work_is_completed(self._h) == _capi.OK

    def wait(self, timeout=None):  # the timeout is ignored, as in the reference
        _capi.check(_capi.lib().frg_work_wait(self._h))
        return True

    def block_stream(self, stream=None):
        import torch
        stream = torch.cuda.current_stream() if stream is None else stream
        _capi.check(_capi.lib().frg_work_block_stream(self._h, stream.cuda_stream))

    def result(self):
        self.wait()
        return [self._keep[0]]

    def __del__(self):
        h, self._h = self._h, None
        if h is not None:
            try:
                _capi.lib().frg_work_release(h)
            except Exception:
                pass


class DeviceFairring:
    def __init__(self, device=0, max_memory_allocated_in_bytes=50 * MiB,
                 max_padding_allocated_in_bytes=MiB, min_parallelism=16,
                 slice_size_in_bytes=0, num_machines=1, num_reduce_streams=0,
                 max_launch_bytes=0, num_copy_streams=0):
        o = _capi.Options(max_memory_allocated_in_bytes, max_padding_allocated_in_bytes,
                          min_parallelism, slice_size_in_bytes, num_machines,
                          num_reduce_streams, num_copy_streams, max_launch_bytes)
        h = ctypes.c_void_p()
        self._h = None
        _capi.check(_capi.lib().frg_create(int(device), ctypes.byref(o), ctypes.byref(h)))
        self._h = h
        self.device = int(device)
        self._reduce_streams = None
        self._copy_streams = None

    def _external_streams(self, getter):
        import torch
        raw = (ctypes.c_void_p * 16)()
        n = ctypes.c_int()
        _capi.check(getter(self._h, raw, 16, ctypes.byref(n)))
        return [torch.cuda.ExternalStream(raw[i], device=self.device)
                for i in range(min(n.value, 16))]

    def _record_on_streams(self, tensors, host=False):
        """Tells torch's caching allocator which of the pipeline's streams touch
        these tensors (the reference does so on its five streams,
        fairring/device.cc:297-301): memory freed while an operation is still
        running is then not handed out again before that stream has passed it.
        The copy streams write `out` when contributions are staged from the host."""
        if self._reduce_streams is None:
                self._reduce_streams = self._external_streams(_capi.lib().frg_get_streams)
        streams = self._reduce_streams
        if host:
            if self._copy_streams is None:
                self._copy_streams = self._external_streams(_capi.lib().frg_get_copy_streams)
            streams = streams + self._copy_streams
        for s in streams:
            for t in tensors:
                if t.is_cuda:
                    t.record_stream(s)

    @property
    def layout(self):
        out = _capi.Layout()
        _capi.check(_capi.lib().frg_get_layout(self._h, ctypes.byref(out)))
        return dict(slot=out.slot_size_in_bytes, slice=out.slice_size_in_bytes,
                    padding_slots=out.num_padding_slots,
                    staging_slots=out.num_staging_slots)

    def _submit(self, out, contribs, op, scale_mode, scale, stream, host, carry=False, done=None):
        import torch
        _check_dense(out, "output")
        for c in contribs:
            if c.numel() != out.numel() or c.dtype != out.dtype:
                raise FairringError(_capi.ERR_INVALID, "contribution shape/dtype mismatch")
        stream = torch.cuda.current_stream(out.device) if stream is None else stream
        tab = _capi.ptr_table([c.data_ptr() for c in contribs])
        wh = ctypes.c_void_p()
        L = _capi.lib()
        head = (self._h, out.data_ptr(), tab, len(contribs), out.numel(), _dtype_code(out), op,
                scale_mode, scale)
        cb = _capi.DONE_FN(done) if done is not None else _capi.DONE_FN()
        tail = (stream.cuda_stream, cb, None, ctypes.byref(wh))
        self._record_on_streams([out] if host else [out] + list(contribs), host=host)
        if host:
            _capi.check(L.frg_allreduce_host(*head, 1 if carry else 0, *tail))
        else:
            _capi.check(L.frg_allreduce(*head, *tail))
        return Work(wh, (out, list(contribs), cb))

    def allreduce(self, out, contribs, op=SUM, scale_mode=SCALE_NONE, scale=1.0, stream=None,
                  done=None):
        """DeviceFairring::allReduce (fairring/device.cc:291-353) with the peers'
        contributions given as GPU tensors. Returns at once. `done(user, status,
        last_stream)`, if given, is the completion callback of frg_allreduce: it
        runs on the pipeline's command thread once the operation is enqueued (or
        on this thread, before the call returns, for a small operation launched
        on the caller's stream)."""
        for c in contribs:
            _check_dense(c, "contribution")
        return self._submit(out, contribs, op, scale_mode, scale, stream, host=False, done=done)

    def allreduce_compressed(self, out, contribs, raw_index=-1, scale_mode=SCALE_NONE, scale=1.0,
                             wire_dtype=None, stream=None, segments=None):
        """reduce_slice_compressed through the slice pipeline (sliced by the
        wire type's element size). With `segments`, the raw fp32 contribution
        is that list of tensors, in the order they lie in the bucket
        (frg_allreduce_compressed_gathered; contribs[raw_index] is ignored and
        may be None, `wire_dtype` must then be given unless there are peers).
        Returns at once."""
        import torch
        _check_dense(out, "output")
        if segments is None:
            for c in contribs:
                _check_dense(c, "contribution")
            wire = _check_compressed(out, contribs, raw_index)
            if wire_dtype is not None:
                wire = BF16 if wire_dtype == torch.bfloat16 else F16
            stream = torch.cuda.current_stream(out.device) if stream is None else stream
            tab = _capi.ptr_table([c.data_ptr() for c in contribs])
            wh = ctypes.c_void_p()
            self._record_on_streams([out] + list(contribs))
            _capi.check(_capi.lib().frg_allreduce_compressed(
                self._h, out.data_ptr(), _dtype_code(out), tab, len(contribs), raw_index,
                out.numel(), wire, scale_mode, scale, stream.cuda_stream, _capi.DONE_FN(), None,
                ctypes.byref(wh)))
            return Work(wh, (out, list(contribs)))
        peers = [c for k, c in enumerate(contribs) if k != raw_index]
        total = 0
        for t in segments:
            _check_dense(t, "segment")
            if t.dtype != torch.float32 or t.device != out.device:
                raise FairringError(_capi.ERR_INVALID, "segments are fp32 tensors on the output's device")
            total += t.numel()
        if total != out.numel():
            raise FairringError(_capi.ERR_INVALID, "the segments hold %d elements, the output %d"
                                % (total, out.numel()))
        for c in peers:
            _check_dense(c, "contribution")
            if c.numel() != out.numel() or c.dtype not in (torch.bfloat16, torch.float16):
                raise FairringError(_capi.ERR_INVALID, "peers are bf16 / fp16 tensors of the output's length")
        if wire_dtype is None:
            if not peers:
                raise FairringError(_capi.ERR_INVALID, "wire_dtype is required without peers")
            wire_dtype = peers[0].dtype
        wire = BF16 if wire_dtype == torch.bfloat16 else F16
        stream = torch.cuda.current_stream(out.device) if stream is None else stream
        tab = _capi.ptr_table([0 if k == raw_index else c.data_ptr() for k, c in enumerate(contribs)])
        segs = (_capi.Segment * max(1, len(segments)))()
        for i, t in enumerate(segments):
            segs[i].ptr = t.data_ptr()
            segs[i].numel = t.numel()
        wh = ctypes.c_void_p()
        self._record_on_streams([out] + peers + list(segments))
        _capi.check(_capi.lib().frg_allreduce_compressed_gathered(
            self._h, out.data_ptr(), _dtype_code(out), tab, len(contribs), raw_index, segs,
            len(segments), out.numel(), wire, scale_mode, scale, stream.cuda_stream,
            _capi.DONE_FN(), None, ctypes.byref(wh)))
        return Work(wh, (out, peers, list(segments)))

    def allreduce_gathered(self, out, contribs, gathered_index, segments, op=SUM,
                           scale_mode=SCALE_NONE, scale=1.0, stream=None, done=None):
        """allreduce with contribution `gathered_index` given as the list of
        tensors `segments`, in the order they lie in `out` (a bucket's own
        gradients where autograd left them); contribs[gathered_index] is ignored
        and may be None (frg_allreduce_gathered). Returns at once."""
        import torch
        _check_dense(out, "output")
        total = 0
        for t in segments:
            _check_dense(t, "segment")
            if t.dtype != out.dtype:
                raise FairringError(_capi.ERR_INVALID, "segment dtype mismatch")
            total += t.numel()
        if total != out.numel():
            raise FairringError(_capi.ERR_INVALID, "the segments hold %d elements, the output %d"
                                % (total, out.numel()))
        ptrs = []
        for k, c in enumerate(contribs):
            if k == gathered_index:
                ptrs.append(out.data_ptr())
                continue
            _check_dense(c, "contribution")
            if c.numel() != out.numel() or c.dtype != out.dtype:
                raise FairringError(_capi.ERR_INVALID, "contribution shape/dtype mismatch")
            ptrs.append(c.data_ptr())
        stream = torch.cuda.current_stream(out.device) if stream is None else stream
        tab = _capi.ptr_table(ptrs)
        segs = (_capi.Segment * max(len(segments), 1))()
        for i, t in enumerate(segments):
            segs[i].ptr = t.data_ptr()
            segs[i].numel = t.numel()
        wh = ctypes.c_void_p()
        others = [c for k, c in enumerate(contribs) if k != gathered_index]
        self._record_on_streams([out] + others + list(segments))
        cb = _capi.DONE_FN(done) if done is not None else _capi.DONE_FN()
        _capi.check(_capi.lib().frg_allreduce_gathered(
            self._h, out.data_ptr(), tab, len(contribs), gathered_index, segs, len(segments),
            out.numel(), _dtype_code(out), op, scale_mode, scale, stream.cuda_stream, cb, None,
            ctypes.byref(wh)))
        return Work(wh, (out, others, list(segments), cb))

    def allreduce_host(self, out, host_contribs, op=SUM, scale_mode=SCALE_NONE, scale=1.0,
                       carry=False, stream=None):
        """Server-side accumulation of contributions held in pinned host memory;
        with carry=True `out` already holds the first term of the sum."""
        for c in host_contribs:
            _check_dense(c, "contribution", device=False)
            if c.is_cuda or not c.is_pinned():
                raise FairringError(_capi.ERR_INVALID,
                                    "host contributions must be pinned CPU tensors")
        return self._submit(out, host_contribs, op, scale_mode, scale, stream, host=True,
                            carry=carry)

    def prepare(self, out, contribs, op=SUM, scale_mode=SCALE_NONE, scale=1.0, stream=None,
                gathered=None):
        """Validate and marshal an allreduce once; the returned callable submits
        it with a single foreign call (for callers that repeat the same
        operation, e.g. one per DDP bucket per step). The callable returns a
        Work; the tensors stay referenced by the callable and are recorded on
        the pipeline's streams once, here. `gathered` = (index, [tensors]) gives
        that contribution piecewise (allreduce_gathered)."""
        import torch
        _check_dense(out, "output")
        g_index, g_tensors = gathered if gathered is not None else (-1, [])
        ptrs = []
        for k, c in enumerate(contribs):
            if k == g_index:
                ptrs.append(out.data_ptr())
                continue
            _check_dense(c, "contribution")
            if c.numel() != out.numel() or c.dtype != out.dtype:
                raise FairringError(_capi.ERR_INVALID, "contribution shape/dtype mismatch")
            ptrs.append(c.data_ptr())
        stream = torch.cuda.current_stream(out.device) if stream is None else stream
        tab = _capi.ptr_table(ptrs)
        L = _capi.lib()
        others = [c for k, c in enumerate(contribs) if k != g_index]
        if gathered is None:
            fn = L.frg_allreduce
            args = (self._h, ctypes.c_void_p(out.data_ptr()), tab, len(contribs),
                    ctypes.c_int64(out.numel()), _dtype_code(out), op, scale_mode,
                    ctypes.c_float(scale), ctypes.c_void_p(stream.cuda_stream), _capi.DONE_FN(),
                    None)
            keep = (out, others, tab)
        else:
            if sum(t.numel() for t in g_tensors) != out.numel():
                raise FairringError(_capi.ERR_INVALID, "the segments do not add up to the output")
            segs = (_capi.Segment * max(len(g_tensors), 1))()
            for i, t in enumerate(g_tensors):
                _check_dense(t, "segment")
                if t.dtype != out.dtype:
                    raise FairringError(_capi.ERR_INVALID, "segment dtype mismatch")
                segs[i].ptr = t.data_ptr()
                segs[i].numel = t.numel()
            fn = L.frg_allreduce_gathered
            args = (self._h, ctypes.c_void_p(out.data_ptr()), tab, len(contribs), g_index, segs,
                    len(g_tensors), ctypes.c_int64(out.numel()), _dtype_code(out), op, scale_mode,
                    ctypes.c_float(scale), ctypes.c_void_p(stream.cuda_stream), _capi.DONE_FN(),
                    None)
            keep = (out, others, tab, segs, list(g_tensors))
        self._record_on_streams([out] + others + list(g_tensors))

        def submit():
            wh = ctypes.c_void_p()
            rc = fn(*args, ctypes.byref(wh))
            if rc != _capi.OK:
                _capi.check(rc)
            return Work(wh, keep)

        return submit

    def progress(self):
        """Operations submitted / started / fully enqueued, kernel launches
        issued, operations launched by the call itself on the producer stream
        (small ones, with nothing in flight), operations run as one with others
        that were waiting in the queue, and launches that covered pieces of
        several such operations, so far."""
        out = (ctypes.c_int64 * 7)()
        _capi.check(_capi.lib().frg_get_progress2(self._h, ctypes.byref(out), ctypes.sizeof(out)))
        return dict(submitted=out[0], started=out[1], enqueued=out[2], launches=out[3],
                    on_callers_stream=out[4], merged=out[5], segmented_launches=out[6])

    def synchronize(self):
        _capi.check(_capi.lib().frg_synchronize(self._h))

    def set_profiling(self, per_launch):
        """Per-launch dispatch timestamps on or off."""
        _capi.check(_capi.lib().frg_set_profiling(self._h, 1 if per_launch else 0))

    def profile_mark(self):
        """One timing event on every reduce stream, in submission order; two
        marks bracket a region that launch_records() reports per stream."""
        _capi.check(_capi.lib().frg_profile_mark(self._h))

    def kernel_times_ms(self, capacity=1 << 16):
        buf = (ctypes.c_float * capacity)()
        n = ctypes.c_int()
        _capi.check(_capi.lib().frg_kernel_times(self._h, buf, capacity, ctypes.byref(n)))
        return list(buf[:min(n.value, capacity)])

    def launch_records(self, capacity=1 << 16):
        """(begin_ms, end_ms, numel, K, stream_index, launches) of every record."""
        buf = (_capi.LaunchRecord * capacity)()
        n = ctypes.c_int()
        _capi.check(_capi.lib().frg_launch_records(self._h, buf, capacity, ctypes.byref(n)))
        return [(r.begin_ms, r.end_ms, r.numel, r.num_contributions, r.stream_index, r.launches)
                for r in buf[:min(n.value, capacity)]]

    def close(self):
        h, self._h = self._h, None
        if h is not None:
            _capi.lib().frg_destroy(h)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
