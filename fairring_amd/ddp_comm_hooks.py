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

__all__ = ["allreduce_hook", "fp16_compress_hook", "bf16_compress_hook"]


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


def _compress_hook(dtype, process_group, bucket):
    buf = bucket.buffer()
    work = _backend(process_group, buf.device)._allreduce_compressed(buf, dtype)
    return work.get_future().then(_first)


def fp16_compress_hook(process_group, bucket):
    """fp16_compress_hook (default_hooks.py:96-113): the bucket cast to float16
    and divided by the group size, summed, and copied back into the bucket."""
    return _compress_hook(torch.float16, process_group, bucket)


def bf16_compress_hook(process_group, bucket):
    """bf16_compress_hook (default_hooks.py:116-134), as above with bfloat16."""
    return _compress_hook(torch.bfloat16, process_group, bucket)
