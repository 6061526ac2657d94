"""The plug-in boundary: the wrappers Merak's module rebuild instantiates.

``build_layers`` has the signature of Merak/core/tensor_parallel/mp_layers.py:507-536
and is keyed on the ``mp_attr`` tag that ``set_mp_attr`` (mp_attrs.py:43-147) leaves
on a module; ``ColPara`` / ``RowPara`` mirror :74-184 at ``tp_overlapping_level``
0 (the async / piped variants only reorder communication, which does not exist
on one GPU).  State-dict keys stay ``<name>.col_linear.{weight,bias}`` and
``<name>.row_linear.{weight,bias}``.
"""
from __future__ import annotations

from typing import Callable

import torch
import torch.nn as nn

from .. import mpu
from ..args import get_args


def _require_level0():
    level = getattr(get_args(), "tp_overlapping_level", 0)
    if level != 0:
        raise NotImplementedError(
            f"tp_overlapping_level={level}: the communication-overlap variants (mp_layers.py:194-504) only matter "
            "with more than one tensor-parallel rank and are not part of this build; use level 0")


class ColPara(torch.nn.Module):
    def __init__(self, in_feature, out_feature, init_method, bias=True, gather_output=False, need_permute=False):
        super().__init__()
        self.need_permute = need_permute
        _require_level0()
        self.col_linear = mpu.ColumnParallelLinear(
            in_feature,
            out_feature,
            bias=bias,
            gather_output=gather_output,
            init_method=init_method,
            skip_bias_add=False)

    @property
    def weight(self):
        return self.col_linear.weight

    @property
    def bias(self):
        return self.col_linear.bias

    def forward(self, x):
        # (batch, seq, hidden) -> (seq, batch, hidden) when asked to (mp_layers.py:115-126)
        if self.need_permute:
            x = x.permute(1, 0, 2)
        intermediate_parallel, _ = self.col_linear(x)
        if self.need_permute:
            return intermediate_parallel.permute(1, 0, 2)
        return intermediate_parallel


class RowPara(torch.nn.Module):
    def __init__(self, in_feature, out_feature, output_layer_init_method, bias=True, input_is_parallel=True,
                 need_permute=False):
        super().__init__()
        self.need_permute = need_permute
        _require_level0()
        self.return_bias = False  # True only for overlap level > 1 (mp_layers.py:135)
        self.row_linear = mpu.RowParallelLinear(
            in_feature,
            out_feature,
            bias=bias,
            input_is_parallel=input_is_parallel,
            init_method=output_layer_init_method,
            skip_bias_add=False)

    @property
    def weight(self):
        return self.row_linear.weight

    @property
    def bias(self):
        return self.row_linear.bias

    def forward(self, x):
        if self.need_permute:
            x = x.permute(1, 0, 2)
        output, bias = self.row_linear(x)
        if self.need_permute:
            return output.permute(1, 0, 2)
        if self.return_bias:
            return output, bias
        return output


def build_layers(name: str, module: torch.nn.Module, mp_size: int, init_method: Callable,
                 scaled_init_method: Callable):
    """Tagged ``nn.Linear`` / HF ``Conv1D`` -> ``ColPara`` / ``RowPara`` with the *global* sizes restored
    (mp_layers.py:507-531).  Untagged linears come back unchanged; anything else gives ``None``.
    Conv2d tensor parallelism (``ConvPara``) is outside this build."""
    if isinstance(module, nn.Linear) or name in ['c_attn', 'c_proj', 'c_fc']:
        _bias = module.bias if isinstance(module.bias, bool) else isinstance(module.bias, torch.Tensor)
        if not hasattr(module, 'mp_attr'):
            return module
        elif module.mp_attr.startswith('row'):
            module_args = [module.in_features * mp_size, module.out_features]
            return RowPara(module_args[0], module_args[1], scaled_init_method, bias=_bias, need_permute=False)
        elif module.mp_attr.startswith('col'):
            module_args = [module.in_features, module.out_features * mp_size]
            return ColPara(module_args[0], module_args[1], init_method, bias=_bias, need_permute=False)
        return None
    elif isinstance(module, nn.Conv2d):
        if not hasattr(module, 'mp_attr'):
            return module
        raise NotImplementedError("ConvPara (conv tensor parallelism, mp_layers.py:33-72) is outside this build")
    else:
        return None
