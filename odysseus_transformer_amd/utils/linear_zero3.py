"""Linear layer whose weight is a ZeRO-3 row shard (utils/linear_zero3.py of the
reference): the full weight is gathered for every use and the full weight gradient is
reduce-scattered back to the shard.  At world_size = 1 the shard is the full weight;
the products run on the HIP library.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from ..parallel_state import (get_model_parallel_group, get_model_parallel_world_size, require_single_rank)
from .comm import prepare_input_tensors_for_wgrad_compute
from .linear_tpsp import linear_dgrad, linear_forward, linear_wgrad


def _gather_weight(weight: torch.Tensor) -> torch.Tensor:
    """Row shards (out / N, in) -> (out, in) (utils/linear_zero3.py:35-43, :58-65)."""
    if get_model_parallel_world_size() == 1:
        return weight
    require_single_rank("all-gather of the ZeRO-3 weight shards")


def _reduce_scatter_weight_grad(grad_weight_global: torch.Tensor) -> torch.Tensor:
    """(out, in) summed over ranks -> this rank's (out / N, in) rows (utils/linear_zero3.py:76-84)."""
    if get_model_parallel_world_size() == 1:
        return grad_weight_global
    require_single_rank("reduce-scatter of the ZeRO-3 weight gradient")


class LinearZeROFunc(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, input, weight, bias):
        ctx.save_for_backward(input, weight)
        ctx.use_bias = bias is not None
        return linear_forward(input, _gather_weight(weight), bias)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        input, weight = ctx.saved_tensors
        full_weight = _gather_weight(weight)
        grad_input = linear_dgrad(grad_output, full_weight)
        g2, x2 = prepare_input_tensors_for_wgrad_compute(grad_output, input)
        grad_weight = _reduce_scatter_weight_grad(linear_wgrad(g2, x2))
        grad_bias = g2.sum(dim=0) if ctx.use_bias else None
        return grad_input, grad_weight, grad_bias


def linear_with_zero(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    return LinearZeROFunc.apply(input, weight, bias)


class LinearZeRO3(nn.Module):
    """weight (output_features // N, input_features); as in the reference it is left
    uninitialised (utils/linear_zero3.py:113-115): the owner loads or initialises it."""

    def __init__(self, input_features, output_features, bias=False):
        super().__init__()
        self.input_features = input_features
        self.output_features = output_features
        self.world_size = get_model_parallel_world_size()
        self.group = get_model_parallel_group()
        self.weight = nn.Parameter(torch.empty(output_features // self.world_size, input_features))
        if bias:
            self.bias = nn.Parameter(torch.empty(output_features // self.world_size))
        else:
            self.register_parameter("bias", None)

    def forward(self, input):
        return linear_with_zero(input=input, weight=self.weight, bias=self.bias)
