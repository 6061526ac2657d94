"""Model-parallel random number states (what Merak/core/recompute/checkpointing.py:106-252 keeps for the
tensor-parallel layers): a named generator state per purpose, swapped in for the duration of a ``with`` block.

``model_parallel_manual_seed(seed)`` seeds the default generator with ``seed`` (the same on every rank of a
tensor-parallel group) and registers the state ``'model-parallel-rng'`` seeded with ``seed + 2718 + rank``
(different on every rank of the group, checkpointing.py:213-221 without the sequence-parallel axis, which one GPU
does not have).  ``_initialize_affine_weight_gpu`` draws a shard's initial values under that state
(Merak/core/mpu/layers.py:52-53), so that shard-building ranks with one seed get different shards."""
import contextlib

import torch

from .initialize import get_model_parallel_rank

MODEL_PARALLEL_RNG = "model-parallel-rng"


def _get_state():
    """(CPU generator state, current GPU's generator state or None): a shard may be drawn on either device
    (use_cpu_initialization builds it on the host, the device path on the GPU), so both are tracked."""
    return (torch.get_rng_state(), torch.cuda.get_rng_state() if torch.cuda.is_available() else None)


def _set_state(state):
    cpu, gpu = state
    torch.set_rng_state(cpu)
    if gpu is not None and torch.cuda.is_available():
        torch.cuda.set_rng_state(gpu)


def _seed(seed):
    # torch.manual_seed seeds the CPU generator and every GPU's
    torch.manual_seed(seed)


class RNGStatesTracker:
    """Named generator states.  ``add(name, seed)`` registers one; ``fork(name)`` makes it the current state inside
    a ``with`` block and stores where it got to on the way out."""

    def __init__(self):
        self.reset()

    def reset(self):
        self._states = {}
        self._seeds = set()

    def get_states(self):
        return dict(self._states)

    def set_states(self, states):
        self._states = states

    def has(self, name=MODEL_PARALLEL_RNG):
        return name in self._states

    def add(self, name, seed):
        if seed in self._seeds:
            raise Exception("seed {} already exists".format(seed))
        if name in self._states:
            raise Exception("cuda rng state {} already exists".format(name))
        self._seeds.add(seed)
        outer = _get_state()
        _seed(seed)
        self._states[name] = _get_state()
        _set_state(outer)

    @contextlib.contextmanager
    def fork(self, name=MODEL_PARALLEL_RNG):
        if name not in self._states:
            raise Exception("cuda rng state {} is not added".format(name))
        outer = _get_state()
        _set_state(self._states[name])
        try:
            yield
        finally:
            self._states[name] = _get_state()
            _set_state(outer)


_TRACKER = RNGStatesTracker()


def get_rng_tracker():
    return _TRACKER


def model_parallel_manual_seed(seed):
    """Call after the tensor-parallel size and rank are set (checkpointing.py:196-252)."""
    _TRACKER.reset()
    _seed(seed)
    _TRACKER.add(MODEL_PARALLEL_RNG, seed + 2718 + get_model_parallel_rank())
