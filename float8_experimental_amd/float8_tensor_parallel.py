"""Tensor-parallel styles of the reference (``float8_tensor_parallel.py``: ``Float8ColwiseParallel``,
``Float8RowwiseParallel``, ``PrepareFloat8ModuleInput``) shard a layer over several GPUs with DTensor and move
fp8 bytes in the all-gather.  This build drives one GPU and has no collectives; the names exist so that an
import written for the reference fails with a sentence instead of a ``ModuleNotFoundError``.  The per-GPU
work of those styles is the same path as everywhere else here: cast the local activation to fp8 before the
gather (``float8_tensor_parallel.py:49-61``), multiply the local weight slice.
"""


class _NeedsSeveralGPUs:
    def __init__(self, *args, **kwargs):
        raise NotImplementedError(
            f"{type(self).__name__} shards a layer over several GPUs (DTensor tensor parallelism with a float8 "
            "all-gather); this build drives a single MI355X and has no collectives")


class Float8ColwiseParallel(_NeedsSeveralGPUs):
    pass


class Float8RowwiseParallel(_NeedsSeveralGPUs):
    pass


class PrepareFloat8ModuleInput(_NeedsSeveralGPUs):
    pass
