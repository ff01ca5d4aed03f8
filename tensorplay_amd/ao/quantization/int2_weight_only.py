"""INT2 weight-only Linear (reference: tensorplay/ao/quantization/int2_weight_only.py).

Symmetric group-wise 2-bit codes {0..3} standing for {-2, -1, 0, 1} * scale, four per byte with the
first code in the two most significant bits; buffers as in the reference (``weight`` uint8
[N, ceil(K/4)], ``scales_and_zeros`` float32 [K/g, N, 2]).  The forward is one HIP kernel on the packed
bytes.  The straight-through training linear is not built.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

import torch
import torch.nn as nn

from ... import ops
from .intx_weight_only import _packed_linear
from .quantize_api import quantize_, register_quantize_module_handler


def _quantize_int2_groupwise(weight: torch.Tensor, groupsize: int,
                             eps: float = 1e-8) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(codes int8 [N, K] in {0..3}, scale, zero [N, K/g]); scale = max|w| / 2, zero = 2 (reference :41-60)."""
    N, K = weight.shape
    if K % groupsize != 0:
        raise ValueError(f"int2 weight-only requires K={K} divisible by groupsize={groupsize}")
    w = weight.reshape(N, K // groupsize, groupsize)
    scale = (w.abs().amax(dim=-1) / 2.0).clamp(min=eps)
    codes = ((w / scale.unsqueeze(-1)).round() + 2.0).clamp(0, 3).to(torch.int8).reshape(N, K)
    return codes, scale, torch.full_like(scale, 2.0)


def pack_int2(codes: torch.Tensor) -> torch.Tensor:
    """Four 2-bit codes per byte, the first in the two most significant bits (reference :63-88)."""
    return ops.pack_lowbit(codes, 2)


def unpack_int2(packed: torch.Tensor, columns: int) -> torch.Tensor:
    """uint8 codes {0..3} [..., columns] (reference :91-103)."""
    return ops.unpack_lowbit(packed, 2, columns)


def _pack_int2_weight(weight: torch.Tensor, groupsize: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """(packed uint8, scale_zero [K/g, N, 2]) of a float weight (reference :106-112)."""
    codes, scale, zero = _quantize_int2_groupwise(weight, groupsize)
    return pack_int2(codes), torch.stack([scale.t(), zero.t()], dim=-1).contiguous()


def _dequantize_int2(packed: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor, columns: int) -> torch.Tensor:
    """float32 [N, K] = (code - zero) * scale (reference :115-129)."""
    return ops._lowbit_dequantize(packed, 2, columns, torch.stack([scale.t(), zero.t()], dim=-1), torch.float32)


def _int2_mm(input: torch.Tensor, packed: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor, columns: int) -> torch.Tensor:
    """INT2 matmul with scale, zero [N, K/g] (reference :132-139)."""
    return _packed_linear(input, packed, 2, columns, torch.stack([scale.t(), zero.t()], dim=-1), None)


class WeightOnlyInt2Linear(nn.Module):
    """Inference linear with a packed INT2 weight and per-group scales (reference :142-223).
    ``cache_unpacked`` is accepted and ignored: the kernel reads the packed bytes."""

    def __init__(self, in_features: int, out_features: int, groupsize: int = 128, bias: bool = False,
                 cache_unpacked: bool = False, device=None):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.groupsize = groupsize
        self.cache_unpacked = cache_unpacked
        self.register_buffer("weight", torch.zeros((out_features, (in_features + 3) // 4), dtype=torch.uint8, device=device))
        self.register_buffer("scales_and_zeros",
                             torch.zeros((in_features // groupsize, out_features, 2), dtype=torch.float32, device=device))
        if bias:
            self.register_buffer("bias", torch.zeros(out_features, dtype=torch.float32, device=device))
        else:
            self.bias = None

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        act_pre_scale = getattr(self, "act_pre_scale", None)
        if act_pre_scale is not None:
            input = input * act_pre_scale
        return _packed_linear(input, self.weight, 2, self.in_features, self.scales_and_zeros, self.bias)

    @classmethod
    def from_float(cls, linear: nn.Linear, groupsize: int = 128, cache_unpacked: bool = False) -> "WeightOnlyInt2Linear":
        if linear.bias is not None and linear.bias.dim() != 1:
            raise ValueError("int2 weight-only requires a 1-D bias or no bias")
        w = linear.weight.detach()
        # quantized in the weight's own dtype, as the reference does (:207); the kernel reads float32 parameters
        packed, scale_zero = _pack_int2_weight(w, groupsize)
        scale_zero = scale_zero.float()
        mod = cls(linear.in_features, linear.out_features, groupsize=groupsize, bias=linear.bias is not None,
                  cache_unpacked=cache_unpacked, device=w.device)
        mod.weight = packed
        mod.scales_and_zeros = scale_zero
        if linear.bias is not None:
            mod.bias = linear.bias.detach().float()
        return mod


@dataclass
class Int2WeightOnlyConfig:
    """groupsize: number of input columns sharing one scale/zero."""

    groupsize: int = 128


int2_weight_only = Int2WeightOnlyConfig


@register_quantize_module_handler(Int2WeightOnlyConfig)
def _int2_weight_only_transform(module, config):
    """Replace an ``nn.Linear`` with a packed INT2 weight-only linear (reference :291-297)."""
    cache = getattr(module, "_int2_cache_unpacked", False)
    return WeightOnlyInt2Linear.from_float(module, config.groupsize, cache_unpacked=cache)


def quantize_int2_weight_only(model: nn.Module, groupsize: int = 128) -> nn.Module:
    return quantize_(model, int2_weight_only(groupsize=groupsize))
