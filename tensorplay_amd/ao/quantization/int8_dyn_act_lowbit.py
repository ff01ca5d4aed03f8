"""int8 dynamic-activation linears with int4 / int2 / 1-bit weights (reference:
tensorplay/ao/quantization/int8_dyn_act_int4_weight.py, int8_dyn_act_int2_weight.py,
int8_dyn_act_int1_weight.py).

Forward, as in the reference: the activations are quantized per token to int8, the full-precision weight
per row to signed 4 / 2 / 1-bit codes by the fused native quantizers, the product runs on the int8
matrix cores and is rescaled by both scales.  Backward is the reference's straight-through estimator
(plain matmuls on the full-precision weight), so the modules stay trainable.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn as nn

from ... import ops
from .bitnet import quantize_int8_rowwise
from .int8_mixed_precision import _int8_mm
from .quantize_api import register_quantize_module_handler


def _quantize_int4_weight_signed(weight: torch.Tensor):
    """(codes int8 [N, K] in [-8, 7], scale [N] = max|w| / 7) (reference int8_dyn_act_int4_weight.py:44-69, device branch)."""
    return ops._quantize_int4_rowwise(weight, 1e-8)


def _quantize_int2_weight_signed(weight: torch.Tensor):
    """(codes int8 in [-2, 1], scale [N] = max|w| / 2) (reference int8_dyn_act_int2_weight.py:28-34)."""
    return ops._quantize_int2_rowwise(weight, 1e-8)


def _quantize_binary_weight_signed(weight: torch.Tensor):
    """(codes int8 in {-1, +1}, scale [N] = max|w|) (reference int8_dyn_act_int1_weight.py:27-34)."""
    return ops._quantize_binary_rowwise(weight, 1e-8)


class _Int8DynActLowBitLinear(torch.autograd.Function):
    """Quantized forward, straight-through backward (reference int8_dyn_act_int4_weight.py:72-95)."""

    @staticmethod
    def forward(ctx, input, weight, quantize_weight):
        flat = input.reshape(-1, input.shape[-1])
        x_i8, x_scale = quantize_int8_rowwise(flat.detach())
        w_codes, w_scale = quantize_weight(weight.detach())
        ctx.save_for_backward(input, weight)
        out = _int8_mm(x_i8, w_codes, x_scale, w_scale)
        return out.reshape(*input.shape[:-1], out.shape[-1])

    @staticmethod
    def backward(ctx, grad_output):
        input, weight = ctx.saved_tensors
        grad_weight = grad_output.reshape(-1, weight.shape[0]).T @ input.reshape(-1, weight.shape[1])
        grad_input = grad_output @ weight.to(grad_output.dtype)
        return grad_input, grad_weight, None


class Int8DynActInt4WeightLinear(nn.Linear):
    """Linear with int8 dynamic activations and int4 weights (reference :98-108).  ``groupsize`` is kept
    for configuration compatibility: the weight scale is per row, as in the reference."""

    def __init__(self, *args, groupsize: int = 128, **kwargs):
        super().__init__(*args, **kwargs)
        self.groupsize = groupsize

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return _Int8DynActLowBitLinear.apply(input, self.weight, _quantize_int4_weight_signed)


class Int8DynActInt2WeightLinear(nn.Linear):
    """Linear with int8 dynamic activations and int2 weights (reference int8_dyn_act_int2_weight.py:60-71)."""

    def __init__(self, *args, groupsize: int = 128, **kwargs):
        super().__init__(*args, **kwargs)
        self.groupsize = groupsize

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return _Int8DynActLowBitLinear.apply(input, self.weight, _quantize_int2_weight_signed)


class Int8DynActBinaryWeightLinear(nn.Linear):
    """Linear with int8 dynamic activations and 1-bit weights (reference int8_dyn_act_int1_weight.py:59-64)."""

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return _Int8DynActLowBitLinear.apply(input, self.weight, _quantize_binary_weight_signed)


@dataclass
class Int8DynamicActivationInt4WeightConfig:
    groupsize: int = 128


@dataclass
class Int8DynamicActivationInt2WeightConfig:
    groupsize: int = 128


@dataclass
class Int8DynamicActivationBinaryWeightConfig:
    pass


int8_dynamic_activation_int4_weight = Int8DynamicActivationInt4WeightConfig
int8_dynamic_activation_int2_weight = Int8DynamicActivationInt2WeightConfig
int8_dynamic_activation_binary_weight = Int8DynamicActivationBinaryWeightConfig


@register_quantize_module_handler(Int8DynamicActivationInt4WeightConfig)
def _int8_dyn_act_int4_transform(module, config):
    module.__class__ = Int8DynActInt4WeightLinear
    module.groupsize = config.groupsize
    return module


@register_quantize_module_handler(Int8DynamicActivationInt2WeightConfig)
def _int8_dyn_act_int2_transform(module, config):
    module.__class__ = Int8DynActInt2WeightLinear
    module.groupsize = config.groupsize
    return module


@register_quantize_module_handler(Int8DynamicActivationBinaryWeightConfig)
def _int8_dyn_act_binary_transform(module, config):
    module.__class__ = Int8DynActBinaryWeightLinear
    return module
