"""Weight-init closures Merak hands to the layers (Merak/core/tensor_parallel/utils.py:30-47)."""
from __future__ import annotations

import math
from typing import Callable, Union

import torch


def init_method_normal(sigma: float) -> Callable:
    """Init method based on N(0, sigma)."""
    def init_(tensor: torch.Tensor) -> torch.Tensor:
        return torch.nn.init.normal_(tensor, mean=0.0, std=sigma)

    return init_


def scaled_init_method_normal(sigma: float, num_layers: Union[int, dict]) -> Callable:
    """Init method based on N(0, sigma / sqrt(2 * num_layers))."""
    if isinstance(num_layers, dict):
        num_layers = sum(list(num_layers.values()))
    std = sigma / math.sqrt(2.0 * num_layers)

    def init_(tensor: torch.Tensor) -> torch.Tensor:
        return torch.nn.init.normal_(tensor, mean=0.0, std=std)

    return init_
