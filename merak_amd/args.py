"""The handful of global arguments the tensor-parallel layers read at
construction time.

In the reference these come from ``Merak.merak_args.get_args()``
(Merak/merak_args/args.py:581-592): ``params_dtype`` (fp16 or fp32 there; bf16
is applied afterwards by ``module.bfloat16()``, Merak/core/amp/amp_engine.py:130-139),
``use_cpu_initialization``, ``use_cpu`` and ``tp_overlapping_level``.  This
module keeps the same ``get_args()`` accessor so the layer code reads like the
reference's; ``set_args`` replaces the global, and any object with those
attributes (a real ``MerakArguments`` included) can be installed.
"""
from __future__ import annotations

from types import SimpleNamespace

import torch

_DEFAULTS = dict(
    params_dtype=torch.float32,       # args.py:584-587
    use_cpu_initialization=False,     # args.py:588-589 (True when no accelerator is used)
    use_cpu=False,
    tp_overlapping_level=0,           # only level 0 (plain layers) exists here
    parallel_vocab=False,
    init_method_std=0.02,
    num_layers=1,
    seed=1234,
)

_ARGS = SimpleNamespace(**_DEFAULTS)


def get_args():
    return _ARGS


def set_args(obj=None, **overrides):
    """Install ``obj`` (or a fresh default namespace) as the global args, then apply overrides."""
    global _ARGS
    if obj is None:
        obj = SimpleNamespace(**_DEFAULTS)
    for k, v in _DEFAULTS.items():
        if not hasattr(obj, k):
            setattr(obj, k, v)
    for k, v in overrides.items():
        setattr(obj, k, v)
    _ARGS = obj
    return _ARGS
