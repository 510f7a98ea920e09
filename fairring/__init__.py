"""Drop-in plugin: ``import fairring`` registers the c10d backend "fairring".

    import fairring
    torch.distributed.init_process_group("fairring", ...)

Mirrors fairring/__init__.py:17-49 of the reference: the staging options come
from FAIRRING_TOTAL_MEMORY / FAIRRING_PADDING_MEMORY / FAIRRING_PARALLELISM
(and the README's FAIRRING_SLICE_SIZE), and the process group is the compiled
``_fairring.ProcessGroup`` (here built from fairring_amd/csrc/torch_ext).
"""
import sys

import torch.distributed

# Must come after torch
from fairring_amd import _fairring  # isort: skip
from fairring_amd.device import options_from_env

sys.modules.setdefault("_fairring", _fairring)


def create_process_group_fairring(store, rank, size, timeout):
    opts = options_from_env()
    return _fairring.ProcessGroup(
        store,
        rank,
        size,
        _fairring.ProcessGroup.Options(
            max_memory_allocated_in_bytes=opts["max_memory_allocated_in_bytes"],
            max_padding_allocated_in_bytes=opts["max_padding_allocated_in_bytes"],
            min_parallelism=opts["min_parallelism"],
            is_high_priority_stream=True,
            timeout=timeout,
            slice_size_in_bytes=opts.get("slice_size_in_bytes", 0),
        ),
    )


torch.distributed.Backend.register_backend(
    "fairring", create_process_group_fairring, devices=["cuda"])
