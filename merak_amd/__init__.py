"""merak_amd — gfx950 (MI355X) kernels behind Merak's Megatron-style
tensor-parallel layers, with the reference's module / function surface.

    from merak_amd import mpu
    layer = mpu.ColumnParallelLinear(4096, 6144, bias=False, gather_output=False)

The compute lives in ``merak_amd/lib/libmerak_tp_gfx950.so`` (C ABI in
``include/merak_tp_gfx950.h``; build with ``python -m merak_amd.build``).
"""
from . import mpu  # noqa: F401
from .args import get_args, set_args  # noqa: F401

__version__ = "0.1.0"
