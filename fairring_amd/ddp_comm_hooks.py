"""DDP communication hooks with the hook's arithmetic folded into the reduction.

Same names, signatures and results as torch's own hooks
(torch:distributed/algorithms/ddp_comm_hooks/default_hooks.py), for a process
group of the "fairring" backend:

    ddp_model.register_comm_hook(process_group, fairring_amd.ddp_comm_hooks.bf16_compress_hook)

torch's hooks run separate passes over every bucket around the allreduce (a
division; or a cast, a division and a copy back). These hand the raw bucket to
the backend, whose reduction kernel does the same arithmetic in registers:
the bucket crosses HBM once on the way in and once on the way out.
"""
import torch
import torch.distributed as dist

__all__ = ["allreduce_hook", "allreduce_from_grads_hook", "fp16_compress_hook",
           "bf16_compress_hook", "fp16_compress_from_grads_hook", "bf16_compress_from_grads_hook"]


def _backend(process_group, device):
    group = process_group if process_group is not None else dist.group.WORLD
    backend = group._get_backend(device) if hasattr(group, "_get_backend") else group
    if not hasattr(backend, "_allreduce_compressed"):
        raise RuntimeError("these hooks need a process group of the 'fairring' backend, got %r"
                           % (backend,))
    return backend


def _first(fut):
    return fut.value()[0]


def allreduce_hook(process_group, bucket):
    """allreduce_hook (default_hooks.py:35-54): the mean over the group, every
    rank's bucket divided by the group size before the sum."""
    buf = bucket.buffer()
    return _backend(process_group, buf.device)._allreduce_pre_divided(buf).get_future().then(_first)


def allreduce_from_grads_hook(process_group, bucket):
    """allreduce_hook for a model wrapped with DDP's default
    gradient_as_bucket_view=False: this rank's contribution is read from the
    parameters' .grad tensors, where autograd left them, instead of from the
    bucket the reducer has copied them into, and the reduced mean is written to
    the bucket once. Same result as allreduce_hook, bit for bit. (The reducer
    still makes its copy before it calls any hook; what this hook shows is the
    reduction that makes that copy unnecessary, for a reducer that skips it.)
    Falls back to allreduce_hook when a gradient is missing, is a view into the
    bucket already, or is not laid out like its place in the bucket."""
    buf = bucket.buffer()
    backend = _backend(process_group, buf.device)
    grads = _grads_apart_from(bucket, buf)
    if grads is None:
        return backend._allreduce_pre_divided(buf).get_future().then(_first)
    return backend._allreduce_from_grads(buf, grads, True).get_future().then(_first)


def _grads_apart_from(bucket, buf):
    """The parameters' .grad tensors where they can stand in for the bucket's
    contents (all there, laid out like their places in the bucket, and not
    views into the bucket already), else None."""
    views = bucket.gradients()
    grads = [p.grad for p in bucket.parameters()]
    usable = len(grads) == len(views) and all(
        g is not None and g.dtype == buf.dtype and g.device == buf.device
        and g.shape == v.shape and g.stride() == v.stride()
        and g.untyped_storage().data_ptr() != buf.untyped_storage().data_ptr()
        for g, v in zip(grads, views))
    if not usable or sum(g.numel() for g in grads) != buf.numel():
        return None
    return grads


def _compress_hook(dtype, process_group, bucket, from_grads=False):
    buf = bucket.buffer()
    backend = _backend(process_group, buf.device)
    grads = _grads_apart_from(bucket, buf) if from_grads and buf.dtype == torch.float32 else None
    if grads is not None:
        work = backend._allreduce_compressed(buf, dtype, grads)
    else:
        work = backend._allreduce_compressed(buf, dtype)
    return work.get_future().then(_first)


def fp16_compress_hook(process_group, bucket):
    """fp16_compress_hook (default_hooks.py:96-113): the bucket cast to float16
    and divided by the group size, summed, and copied back into the bucket."""
    return _compress_hook(torch.float16, process_group, bucket)


def bf16_compress_hook(process_group, bucket):
    """bf16_compress_hook (default_hooks.py:116-134), as above with bfloat16."""
    return _compress_hook(torch.bfloat16, process_group, bucket)


def fp16_compress_from_grads_hook(process_group, bucket):
    """fp16_compress_hook with this rank's contribution read from the
    parameters' .grad tensors (see allreduce_from_grads_hook): cast, division,
    sum and the copy back in one pass over the gradients and the peers' wire
    tensors, the bucket written once. Same result as fp16_compress_hook."""
    return _compress_hook(torch.float16, process_group, bucket, from_grads=True)


def bf16_compress_from_grads_hook(process_group, bucket):
    """bf16_compress_hook likewise."""
    return _compress_hook(torch.bfloat16, process_group, bucket, from_grads=True)
