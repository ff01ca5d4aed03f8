"""1-bit weight-only Linear (reference: tensorplay/ao/quantization/binary.py).

Sign bits {0, 1} standing for {-1, +1} times the row's mean absolute value, eight per byte with code i
in bit i; buffers as in the reference (``weight`` uint8 [N, ceil(K/8)], ``scale`` float32 [N, 1]).  The
forward is the packed n-bit HIP kernel with scale' = 2 scale and zero = 1/2:
(bit - 1/2) * 2 scale = (2 bit - 1) * scale exactly.  The straight-through training linear is not built.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

import torch
import torch.nn as nn

from ... import ops
from .intx_weight_only import _packed_linear
from .quantize_api import quantize_, register_quantize_module_handler


def _quantize_binary_weight(weight: torch.Tensor, eps: float = 1e-8) -> Tuple[torch.Tensor, torch.Tensor]:
    """(sign_bits uint8 [N, K] with 1 for w >= 0, scale [N, 1] = mean |w| per row) (reference :36-47)."""
    scale = weight.abs().mean(dim=-1, keepdim=True).clamp(min=eps)
    return (weight >= 0).to(torch.uint8), scale


def pack_binary(codes: torch.Tensor) -> torch.Tensor:
    """Eight sign codes per byte, code i in bit i (reference :50-71)."""
    return ops.pack_lowbit(codes, 1, lsb_first=True)


def unpack_binary(packed: torch.Tensor, columns: int) -> torch.Tensor:
    """uint8 codes {0, 1} [..., columns] (reference :74-85)."""
    return ops.unpack_lowbit(packed, 1, columns, lsb_first=True)


def _binary_params(scale: torch.Tensor) -> torch.Tensor:
    """[1, N, 2] float32 (2 scale, 1/2) for the packed kernel."""
    s = scale.reshape(-1).to(torch.float32)
    return torch.stack([2.0 * s, torch.full_like(s, 0.5)], dim=-1).unsqueeze(0).contiguous()


def _binary_mm(input: torch.Tensor, packed: torch.Tensor, scale: torch.Tensor, columns: int) -> torch.Tensor:
    """1-bit matmul: input @ ((2 bit - 1) * scale).T (reference :88-95)."""
    return _packed_linear(input, packed, 1, columns, _binary_params(scale), None, lsb_first=True)


class WeightOnlyBinaryLinear(nn.Module):
    """Inference linear with a packed 1-bit weight and per-row scales (reference :98-164).
    ``cache_unpacked`` is accepted and ignored: the kernel reads the packed bytes."""

    def __init__(self, in_features: int, out_features: int, bias: bool = False, cache_unpacked: bool = False, device=None):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.cache_unpacked = cache_unpacked
        self.register_buffer("weight", torch.zeros((out_features, (in_features + 7) // 8), dtype=torch.uint8, device=device))
        self.register_buffer("scale", torch.zeros((out_features, 1), dtype=torch.float32, device=device))
        if bias:
            self.register_buffer("bias", torch.zeros(out_features, dtype=torch.float32, device=device))
        else:
            self.bias = None

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        act_pre_scale = getattr(self, "act_pre_scale", None)
        if act_pre_scale is not None:
            input = input * act_pre_scale
        return _packed_linear(input, self.weight, 1, self.in_features, _binary_params(self.scale), self.bias, lsb_first=True)

    @classmethod
    def from_float(cls, linear: nn.Linear, cache_unpacked: bool = False) -> "WeightOnlyBinaryLinear":
        if linear.bias is not None and linear.bias.dim() != 1:
            raise ValueError("binary weight-only requires a 1-D bias or no bias")
        w = linear.weight.detach()
        sign_bits, scale = _quantize_binary_weight(w)  # in the weight's own dtype, as the reference does (:151)
        scale = scale.float()
        mod = cls(linear.in_features, linear.out_features, bias=linear.bias is not None, cache_unpacked=cache_unpacked,
                  device=w.device)
        mod.weight = pack_binary(sign_bits)
        mod.scale = scale
        if linear.bias is not None:
            mod.bias = linear.bias.detach().float()
        return mod


@dataclass
class BinaryWeightOnlyConfig:
    """Configuration for 1-bit weight-only quantization."""


binary_weight_only = BinaryWeightOnlyConfig


@register_quantize_module_handler(BinaryWeightOnlyConfig)
def _binary_weight_only_transform(module, config):
    """Replace an ``nn.Linear`` with a packed 1-bit weight-only linear (reference :216-220)."""
    cache = getattr(module, "_binary_cache_unpacked", False)
    return WeightOnlyBinaryLinear.from_float(module, cache_unpacked=cache)


def quantize_binary_weight_only(model: nn.Module) -> nn.Module:
    return quantize_(model, binary_weight_only())
