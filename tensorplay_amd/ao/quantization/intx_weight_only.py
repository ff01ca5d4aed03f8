"""n-bit (1..8) weight-only Linear (reference: tensorplay/ao/quantization/intx_weight_only.py).

Same names, packed byte layout (``8 // bits`` codes per byte, the first in the most significant bits)
and buffers (``weight`` uint8 [N, ceil(K / per_byte)], ``scales_and_zeros`` float32 [K/g, N, 2]) as the
reference.  The reference's forward unpacks, dequantizes and calls a float GEMM; here it is one HIP
kernel on the packed bytes (``ops._lowbit_mm``).  The straight-through training linear is not built.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

import torch
import torch.nn as nn

from ... import ops
from .quantize_api import quantize_, register_quantize_module_handler


def pack_intx(codes: torch.Tensor, bits: int) -> torch.Tensor:
    """Pack codes in [0, 2**bits - 1] into uint8 storage (reference :35-59)."""
    return ops.pack_lowbit(codes, bits)


def unpack_intx(packed: torch.Tensor, bits: int, columns: int) -> torch.Tensor:
    """int8 codes [..., columns] (reference :62-80)."""
    return ops.unpack_lowbit(packed, bits, columns).view(torch.int8)


def _quantize_intx_groupwise(weight: torch.Tensor, groupsize: int, bits: int,
                             eps: float = 1e-8) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Affine group-wise n-bit quantization of a 2-D weight (reference :83-107): each group maps its
    minimum to code 0 and its maximum to code 2**bits - 1; returns (codes int8 [N, K], scale, zero
    [N, K/g])."""
    N, K = weight.shape
    if K % groupsize != 0:
        raise ValueError(f"intx weight-only requires K={K} divisible by groupsize={groupsize}")
    groups = K // groupsize
    top = float((1 << bits) - 1)
    w = weight.reshape(N, groups, groupsize)
    min_vals = w.min(dim=-1).values
    max_vals = w.max(dim=-1).values
    scale = ((max_vals - min_vals) / top).clamp(min=eps)
    zero = (-min_vals / scale).round().clamp(0, top)
    codes = ((w - min_vals.unsqueeze(-1)) / scale.unsqueeze(-1)).round().clamp(0, top)
    # codes up to 255 live in the same byte whether it is read as int8 or uint8
    return codes.to(torch.uint8).view(torch.int8).reshape(N, K), scale, zero


def _dequantize_intx(packed: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor, bits: int, columns: int) -> torch.Tensor:
    """float32 [N, K] = (code - zero) * scale; scale, zero [N, K/g] (reference :110-124)."""
    sz = torch.stack([scale.t(), zero.t()], dim=-1)
    return ops._lowbit_dequantize(packed, bits, columns, sz, torch.float32)


def _intx_mm(input: torch.Tensor, packed: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor, bits: int,
             columns: int) -> torch.Tensor:
    """n-bit matmul with scale, zero [N, K/g] (reference :127-133)."""
    sz = torch.stack([scale.t(), zero.t()], dim=-1)
    return _packed_linear(input, packed, bits, columns, sz, None)


def _packed_linear(input, packed, bits, columns, scales_and_zeros, bias, lsb_first=False):
    lead = input.shape[:-1]
    x = input.reshape(-1, input.shape[-1])
    out = ops._lowbit_mm(x, packed, bits, columns, scales_and_zeros, bias, lsb_first)
    return out.reshape(*lead, out.shape[-1])


class WeightOnlyIntxLinear(nn.Module):
    """Inference linear with a packed n-bit weight and per-group scales (reference :136-223).

    ``cache_unpacked`` is accepted for signature parity and ignored: the kernel reads the packed
    bytes directly, so there is no unpacking cost to cache away."""

    def __init__(self, in_features: int, out_features: int, bits: int = 2, groupsize: int = 128, bias: bool = False,
                 cache_unpacked: bool = False, device=None):
        super().__init__()
        if not 1 <= bits <= 8:
            raise ValueError(f"bits must be in [1, 8], got {bits}")
        self.in_features = in_features
        self.out_features = out_features
        self.bits = bits
        self.groupsize = groupsize
        self.cache_unpacked = cache_unpacked
        per_byte = 8 // bits
        self.register_buffer("weight", torch.zeros((out_features, (in_features + per_byte - 1) // per_byte),
                                                   dtype=torch.uint8, device=device))
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
        return _packed_linear(input, self.weight, self.bits, self.in_features, self.scales_and_zeros, self.bias)

    @classmethod
    def from_float(cls, linear: nn.Linear, bits: int = 2, groupsize: int = 128,
                   cache_unpacked: bool = False) -> "WeightOnlyIntxLinear":
        if linear.bias is not None and linear.bias.dim() != 1:
            raise ValueError("intx weight-only requires a 1-D bias or no bias")
        w = linear.weight.detach()
        # quantized in the weight's own dtype, as the reference does (:204-206); the kernel reads float32 parameters
        codes, scale, zero = _quantize_intx_groupwise(w, groupsize, bits)
        scale, zero = scale.float(), zero.float()
        mod = cls(linear.in_features, linear.out_features, bits=bits, groupsize=groupsize, bias=linear.bias is not None,
                  cache_unpacked=cache_unpacked, device=w.device)
        mod.weight = pack_intx(codes, bits)
        mod.scales_and_zeros = torch.stack([scale.t(), zero.t()], dim=-1).contiguous()
        if linear.bias is not None:
            mod.bias = linear.bias.detach().float()
        return mod


@dataclass
class IntxWeightOnlyConfig:
    """bits per weight element in [1, 8]; groupsize: input columns sharing one scale/zero."""

    bits: int = 2
    groupsize: int = 128

    def __post_init__(self):
        if not (1 <= self.bits <= 8):
            raise ValueError(f"bits must be in [1, 8], got {self.bits}")
        if self.groupsize <= 0:
            raise ValueError(f"groupsize must be positive, got {self.groupsize}")


intx_weight_only = IntxWeightOnlyConfig


@register_quantize_module_handler(IntxWeightOnlyConfig)
def _intx_weight_only_transform(module, config):
    """Replace an ``nn.Linear`` with a packed n-bit weight-only linear (reference :288-294)."""
    cache = getattr(module, "_intx_cache_unpacked", False)
    return WeightOnlyIntxLinear.from_float(module, config.bits, config.groupsize, cache_unpacked=cache)


def quantize_intx_weight_only(model: nn.Module, bits: int = 2, groupsize: int = 128) -> nn.Module:
    """Convert every ``nn.Linear`` in ``model`` to n-bit weight-only (reference :296-302)."""
    return quantize_(model, intx_weight_only(bits=bits, groupsize=groupsize))
