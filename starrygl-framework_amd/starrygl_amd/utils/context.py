"""Process context of the single-GPU hot path.

The reference's DistributedContext (starrygl/utils/context.py:28-288) sets up
process groups, a side gloo group, an NCCL id and loggers; the hot path only
ever reads `ctx.device` and `ctx.local_rank` from it (graph.py:44-53, 82).
This class keeps exactly those two, taken from LOCAL_RANK, so that the façade
classes can be constructed the way the reference's callers construct them.
"""
import os


class DistributedContext:
    _default = None

    def __init__(self, device=None, local_rank=None):
        import torch
        if local_rank is None:
            local_rank = int(os.environ.get("LOCAL_RANK", 0))
        if device is None:
            device = torch.device("cuda", local_rank)
        self.device = torch.device(device)
        self.local_rank = int(local_rank)
        self.rank = int(os.environ.get("RANK", 0))
        self.world_size = int(os.environ.get("WORLD_SIZE", 1))

    @classmethod
    def init(cls, backend=None, device=None, local_rank=None, **_unused):
        """One GPU, no process group: `backend` is accepted and ignored."""
        cls._default = cls(device, local_rank)
        return cls._default

    @classmethod
    def get_default_context(cls):
        if cls._default is None:
            cls._default = cls()
        return cls._default
