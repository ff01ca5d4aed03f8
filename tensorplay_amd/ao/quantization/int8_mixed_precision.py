"""Dynamic int8 x int8 linear (reference: tensorplay/ao/quantization/int8_mixed_precision.py:60-100,
229-243).

The reference's device branch runs ``_int_mm`` and then ``_int8_mm_rescale``; ``_int8_mm`` here
produces the same float32 values, ``(float(acc) * row_scale) * col_scale``, in one launch with the
rescale fused into the GEMM epilogue.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn

from ... import ops
from .bitnet import quantize_int8_rowwise
from .quantize_api import register_quantize_module_handler


def _int8_mm(A_i8: torch.Tensor, B_t_i8: torch.Tensor, row_scale: torch.Tensor, col_scale: torch.Tensor) -> torch.Tensor:
    """``(A_i8 @ B_t_i8.T) * row_scale * col_scale`` as float32; A [M,K] int8, B_t [N,K] int8."""
    return ops.int8_mm_dequant(A_i8, B_t_i8, row_scale.reshape(-1), col_scale.reshape(-1))


def scaled_int8_mm(A: torch.Tensor, B: torch.Tensor, row_scale: torch.Tensor, col_scale: torch.Tensor) -> torch.Tensor:
    """``(A @ B) * row_scale * col_scale`` with A [M,K] int8 and B [K,N] int8."""
    return _int8_mm(A, B.t(), row_scale, col_scale)


def _dynamic_int8_mm(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """Quantize ``A`` (any leading dims) and ``B`` ([K,N]) per row / per output channel and multiply."""
    A_i8, A_scale = quantize_int8_rowwise(A.reshape(-1, A.shape[-1]))
    B_t_i8, B_scale = quantize_int8_rowwise(B.T)
    out = _int8_mm(A_i8, B_t_i8, A_scale, B_scale)
    return out.view(*A.shape[:-1], out.shape[-1])


def int8_dynamic_linear(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Forward of the reference's int8 mixed-precision linear (:229-243): the weight is first cast to
    the activation dtype, both operands are quantized per row, and the bias is added afterwards."""
    weight = weight.to(input.dtype)
    out = _dynamic_int8_mm(input, weight.T)
    return out + bias if bias is not None else out


@dataclass
class Int8DynamicLinearConfig:
    """out_dtype: dtype of the module's output (float32 reproduces the reference's two-op result)."""

    out_dtype: torch.dtype = torch.float32


class Int8DynamicLinear(nn.Module):
    """Inference form of the same computation with the weight quantized once: per-channel int8
    codes and scales are buffers, activations are quantized per row on every call, and the
    dequant (and bias) is fused into the GEMM epilogue."""

    def __init__(self, weight_i8: torch.Tensor, weight_scale: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 out_dtype: torch.dtype = torch.float32):
        super().__init__()
        self.out_features, self.in_features = weight_i8.shape
        self.out_dtype = out_dtype
        self.register_buffer("weight", weight_i8.contiguous())
        self.register_buffer("weight_scale", weight_scale.reshape(-1).contiguous())
        if bias is not None:
            self.register_buffer("bias", bias.detach().float().contiguous())
        else:
            self.bias = None

    @classmethod
    def from_float(cls, linear: nn.Linear, out_dtype: torch.dtype = torch.float32) -> "Int8DynamicLinear":
        codes, scale = quantize_int8_rowwise(linear.weight.detach())
        return cls(codes, scale, None if linear.bias is None else linear.bias, out_dtype)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        x = input.reshape(-1, self.in_features)
        x_i8, x_scale = ops._quantize_int8_rowwise(x, 1e-5)
        out = ops.int8_mm_dequant(x_i8, self.weight, x_scale, self.weight_scale, self.bias, self.out_dtype)
        return out.reshape(*input.shape[:-1], self.out_features)


@register_quantize_module_handler(Int8DynamicLinearConfig)
def _int8_dynamic_transform(module, config):
    return Int8DynamicLinear.from_float(module, config.out_dtype)
