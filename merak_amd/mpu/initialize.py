"""Model-parallel world size / rank bookkeeping.

The reference keeps module-global process groups and lets
``set_model_parallel_world_size`` / ``set_model_parallel_rank`` override what
the group would report (Merak/core/mpu/initialize.py:59-84).  The override is
how a single process builds "rank r of p" shards, and it is all this package
needs: one GPU, no collectives.  Without an override the world size is 1 and
the rank 0 (the reference would assert that the group is initialised,
initialize.py:47-48; a lone process has nothing to initialise).
"""
from __future__ import annotations

_MPU_WORLD_SIZE = None
_MPU_RANK = None
_MODEL_PARALLEL_GROUP = None


def set_model_parallel_world_size(world_size):
    """Set the model parallel size (initialize.py:59-62)."""
    global _MPU_WORLD_SIZE
    _MPU_WORLD_SIZE = world_size


def get_model_parallel_world_size() -> int:
    """Return world size for the model parallel group (initialize.py:65-70)."""
    if _MPU_WORLD_SIZE is not None:
        return _MPU_WORLD_SIZE
    return 1


def set_model_parallel_rank(rank):
    """Set model parallel rank (initialize.py:73-76)."""
    global _MPU_RANK
    _MPU_RANK = rank


def get_model_parallel_rank() -> int:
    """Return my rank for the model parallel group (initialize.py:79-84)."""
    if _MPU_RANK is not None:
        return _MPU_RANK
    return 0


def set_model_parallel_group(group):
    """Kept for signature compatibility (initialize.py:151); the group is stored, never used."""
    global _MODEL_PARALLEL_GROUP
    _MODEL_PARALLEL_GROUP = group


def get_model_parallel_group():
    return _MODEL_PARALLEL_GROUP


def destroy_model_parallel():
    global _MPU_WORLD_SIZE, _MPU_RANK, _MODEL_PARALLEL_GROUP
    _MPU_WORLD_SIZE = None
    _MPU_RANK = None
    _MODEL_PARALLEL_GROUP = None
