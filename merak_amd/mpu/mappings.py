"""Identity forms of the tensor-parallel region mappings.

In the reference each mapping is an ``autograd.Function`` around a collective
and each collective is bypassed when the model-parallel world size is 1
(Merak/core/mpu/mappings.py:36,53,89,148).  One GPU, no collectives: only the
bypass exists here.  With a world size above 1 (a process building one rank's
shard) the mappings that would need other ranks' data raise, the ones that are
identities in the direction used do not.
"""
from __future__ import annotations

from .initialize import get_model_parallel_rank, get_model_parallel_world_size
from .utils import split_tensor_along_last_dim


def _needs_peers(name: str):
    raise RuntimeError(
        f"{name}: needs data from other tensor-parallel ranks; this build computes one rank's share on one GPU "
        "and has no collectives (set gather_output=False / input_is_parallel=True, as Merak's wrappers do)")


def copy_to_model_parallel_region(input_):
    """Identity forward (mappings.py:308-321); the backward all-reduce of dX is left to the caller at p > 1."""
    return input_


def reduce_from_model_parallel_region(input_):
    """All-reduce forward (mappings.py:324-337): identity at p == 1; at p > 1 the result is this rank's partial sum."""
    return input_


def scatter_to_model_parallel_region(input_):
    """Keep this rank's slice of the last dimension (mappings.py:47-63); purely local."""
    world_size = get_model_parallel_world_size()
    if world_size == 1:
        return input_
    input_list = split_tensor_along_last_dim(input_, world_size)
    return input_list[get_model_parallel_rank()].contiguous()


def gather_from_model_parallel_region(input_):
    if get_model_parallel_world_size() == 1:
        return input_
    _needs_peers("gather_from_model_parallel_region")
