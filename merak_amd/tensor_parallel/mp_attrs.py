"""Which module becomes which tensor-parallel layer: the feature lists and the tagging pass.

Mirror of Merak/core/tensor_parallel/mp_attrs.py (``set_tp_layer_lists`` :150-202, ``set_mp_attr`` :43-147)
and of the traversal of ``ModuleRebuild.recover_module`` (model_parallel.py:87-99), so that a model can go
through the reference's own sequence - describe the layers, tag them, rebuild them - and land on the gfx950
layers:

    set_tp_layer_lists(col_para_list=[...], row_para_list=[...], ...)
    set_mp_attr(model, mp)                       # tags modules with .mp_attr and divides their sizes
    rebuild_module(model, mp, init, scaled_init) # tagged linears -> ColPara / RowPara

The lists are module-level state, as in the reference.
"""
from __future__ import annotations

from typing import Callable, List, Optional, Tuple

import torch
import torch.nn as nn

from .mp_layers import build_layers

try:  # HF GPT-2's linear ([in, out] weight); the reference reads it from transformers.modeling_utils
    from transformers.pytorch_utils import Conv1D
except Exception:  # pragma: no cover - transformers absent
    class Conv1D:  # type: ignore
        pass

# attributes the reference divides by the tensor-parallel degree when no list is given (:26-27)
DEFAULT_MP_ATTR = ['num_heads', 'split_size', 'n_heads', 'inner_dim']

_lists = {"col": [], "row": [], "conv": [], "weight": [], "io": [], "attr": []}
_lists_set = False


def set_tp_layer_lists(col_para_list: Optional[List[str]] = None, row_para_list: Optional[List[str]] = None,
                       conv_para_list: Optional[List[str]] = None,
                       input_output_mapping: Optional[List[Tuple[int, int, str]]] = None,
                       weight_change_list: Optional[List[Tuple[str, int]]] = None,
                       tp_attr_list: Optional[List[str]] = None):
    """Same arguments and the same requirement as the reference (:181-183): column and row names together, or
    one of the other kinds.  Lists that are not given keep their earlier value (:184-202)."""
    assert (col_para_list and row_para_list) or conv_para_list or weight_change_list or input_output_mapping, \
        'should use at least one kind of tp list to set tp attr'
    global _lists_set
    for key, value in (("col", col_para_list), ("row", row_para_list), ("weight", weight_change_list),
                       ("io", input_output_mapping), ("attr", tp_attr_list), ("conv", conv_para_list)):
        if value:
            _lists[key] = value
    _lists_set = True


def reset_tp_layer_lists():
    """Forget every list (the reference has no such call; tests need one)."""
    global _lists_set
    for key in _lists:
        _lists[key] = []
    _lists_set = False


def get_tp_attr_list() -> List[str]:
    return _lists["attr"]


def mp_is_setted() -> bool:
    return _lists_set


def _tag_linear(m: nn.Module, style: str, mp: int):
    m.mp_attr = style
    if style == 'col':
        m.out_features //= mp
    elif style == 'row':
        m.in_features //= mp


def set_mp_attr(model: nn.Module, mp: int) -> nn.Module:
    """Tags and resizes ``model`` in place for tensor-parallel degree ``mp`` in the reference's order (:44-147):
    column names, row names, the weight-change list, conv names, the in:out ratio table, then the per-module
    attributes (head counts and the like) that are divided by ``mp``."""
    named = list(model.named_modules())
    for key, style in (("col", "col"), ("row", "row")):                       # :44-57
        for n, m in named:
            for part in _lists[key]:
                if part in n and isinstance(m, nn.Linear):
                    _tag_linear(m, style, mp)
    for n, m in named:                                                        # :58-95
        for l_name, d in _lists["weight"]:
            if l_name in n:
                if isinstance(m, nn.Linear):
                    assert d in (0, 1), 'dim should be 0 or 1'
                    _tag_linear(m, 'col' if d == 0 else 'row', mp)
                elif hasattr(m, 'weight'):
                    m.weight.data = m.weight.data.chunk(mp, dim=d)[0].contiguous()
                    if hasattr(m, 'num_embeddings'):
                        m.num_embeddings, m.embedding_dim = m.weight.size(0), m.weight.size(1)
            elif hasattr(m, l_name):
                old = getattr(m, l_name)
                if isinstance(old, nn.Parameter):
                    setattr(m, l_name, nn.Parameter(old.chunk(mp, dim=d)[0].contiguous()))
    for n, m in named:                                                        # :96-101
        if isinstance(m, nn.Conv2d) and any(part in n for part in _lists["conv"]):
            m.mp_attr = 'conv'
    if _lists["io"]:                                                          # :103-130
        for n, m in named:
            if isinstance(m, nn.Linear):
                for i, o, style in _lists["io"]:
                    if m.in_features * o == m.out_features * i:
                        _tag_linear(m, style, mp)
                        break
            elif isinstance(m, Conv1D):
                for i, o, style in _lists["io"]:
                    if m.weight.size(0) * o == m.weight.size(1) * i:
                        m.mp_attr = f'{style}'
                        if style == 'col':
                            m.in_features, m.out_features = m.weight.size(0), m.weight.size(1) // mp
                        elif style == 'row':
                            m.in_features, m.out_features = m.weight.size(0) // mp, m.weight.size(1)
                        break
    attrs = _lists["attr"] or DEFAULT_MP_ATTR                                 # :132-147

    def divide_attrs(parent: nn.Module):
        for n, child in parent.named_children():
            for attr in attrs:
                if hasattr(child, attr):
                    old = getattr(child, attr)
                    assert old % mp == 0, f'mp attr set error, {attr} of {n} is {old}'
                    setattr(child, attr, old // mp)
            if len(list(child.children())) > 0:
                divide_attrs(child)

    divide_attrs(model)
    return model


def rebuild_module(model: nn.Module, mp_size: int, init_method: Callable, scaled_init_method: Callable) -> nn.Module:
    """Replaces, child by child and depth first after the parent, every module ``build_layers`` turns into a
    tensor-parallel layer (the ``build_module`` walk of model_parallel.py:87-99).  Parameters of the new
    layers are freshly initialised; loading a checkpoint is the caller's next step, as in the reference."""
    def walk(parent: nn.Module):
        for n, child in parent.named_children():
            new = build_layers(n, child, mp_size, init_method, scaled_init_method)
            if new is not None:
                setattr(parent, n, new)
            if len(list(child.children())) > 0:
                walk(child)

    walk(model)
    return model
