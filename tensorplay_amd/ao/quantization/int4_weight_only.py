"""int4 weight-only Linear (reference: tensorplay/ao/quantization/int4_weight_only.py:62-201).

Same names, argument order and buffer layout as the reference: ``weight`` holds the device packed
layout int32 [N/8, K/32, 32, 1] written by ``_convert_weight_to_int4pack(codes, 2)`` and
``scales_and_zeros`` is [K/g, N, 2] in the activation dtype.
"""
from __future__ import annotations

import warnings
from dataclasses import dataclass
from typing import Tuple

import torch
import torch.nn as nn

from ... import ops
from .quantize_api import register_quantize_module_handler


@dataclass
class Int4WeightOnlyConfig:
    """groupsize: number of input columns sharing one scale/zero."""

    groupsize: int = 128


int4_weight_only = Int4WeightOnlyConfig


def _quantize_int4_groupwise(weight: torch.Tensor, groupsize: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Symmetric group-wise int4 quantization of a 2-D weight, in the weight's own dtype
    (reference :62-82): scale = max|w| / 8 clamped at 1e-8, codes = clamp(round(w / scale), -8, 7) + 8
    as int32 [N, K]; scale and zero [N, K/g], zero identically 0."""
    N, K = weight.shape
    if K % groupsize != 0:
        raise ValueError(f"int4 weight-only requires K={K} divisible by groupsize={groupsize}")
    groups = K // groupsize
    w = weight.reshape(N, groups, groupsize)
    scale = w.abs().amax(dim=-1) / 8.0
    scale = scale.clamp(min=1e-8)
    codes = (w / scale.unsqueeze(-1)).round().clamp(-8, 7) + 8
    codes = codes.to(torch.int32).reshape(N, K)
    zero = torch.zeros_like(scale)
    return codes, scale, zero


def _pack_int4_weight(weight: torch.Tensor, groupsize: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantize and pack a float weight into (packed int32 device layout, scale_zero [K/g, N, 2])."""
    codes, scale, zero = _quantize_int4_groupwise(weight, groupsize)
    scale_zero = torch.stack([scale.t(), zero.t()], dim=-1).contiguous()
    packed = ops._convert_weight_to_int4pack(codes, 2)
    return packed, scale_zero


def _int4_mm(input: torch.Tensor, packed: torch.Tensor, scale_zero: torch.Tensor, groupsize: int) -> torch.Tensor:
    lead = input.shape[:-1]
    x = input.reshape(-1, input.shape[-1])
    out = ops._weight_int4pack_mm(x, packed, groupsize, scale_zero)
    return out.reshape(*lead, out.shape[-1])


class WeightOnlyInt4Linear(nn.Module):
    """Inference linear with a packed int4 weight and per-group scales (reference :136-184)."""

    def __init__(self, in_features: int, out_features: int, groupsize: int = 128, bias: bool = False,
                 device=None, dtype: torch.dtype = torch.float16):
        super().__init__()
        if in_features % 32 or out_features % 8:
            raise ValueError("WeightOnlyInt4Linear: in_features must be a multiple of 32 and out_features of 8")
        if in_features % groupsize:
            raise ValueError(f"int4 weight-only requires K={in_features} divisible by groupsize={groupsize}")
        self.in_features = in_features
        self.out_features = out_features
        self.groupsize = groupsize
        self.register_buffer("weight", torch.zeros((out_features // 8, in_features // 32, 32, 1), dtype=torch.int32, device=device))
        self.register_buffer("scales_and_zeros",
                             torch.zeros((in_features // groupsize, out_features, 2), dtype=dtype, device=device))
        if bias:
            self.register_buffer("bias", torch.zeros(out_features, dtype=dtype, device=device))
        else:
            self.bias = None

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        act_pre_scale = getattr(self, "act_pre_scale", None)
        if act_pre_scale is not None:
            input = input * act_pre_scale
        out = _int4_mm(input, self.weight, self.scales_and_zeros, self.groupsize)
        if self.bias is not None:
            out = out + self.bias
        return out

    # Layout of a CPU-packed ``weight`` met in a state_dict: (columns per block, half-split nibbles).  The reference's
    # CPU pack depends on the ISA tier it was compiled for (p10/src/backend/cpu/QuantizedElementwiseKernels.cpp:19,
    # 370-390): (64, True) AVX-512 (also what torch's CPU pack writes on such a host), (32, True) AVX2, (32, False)
    # the plain tier.  A state_dict does not say which: set this before load_state_dict.  Left at None, a CPU-layout
    # weight is taken to be the AVX-512 one, with a warning (a pack from another tier would load without error and
    # decode to wrong weights).
    cpu_pack_layout = None

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        """Accepts the module's own buffers (device layout int32 [N/8, K/32, 32, 1]) and the buffers a CPU model of the
        reference saves (reference :150-154, 180-181): ``weight`` uint8 [N, K/2] in the CPU layout, which the device
        op rejects (p10/src/backend/cuda/QuantGemmKernels.cu:1216-1220) and which is converted here on the GPU, and
        ``scales_and_zeros`` [K/g, N, 2] of any float dtype (float32 placeholders included), cast to the module's."""
        key = prefix + "weight"
        w = state_dict.get(key)
        if isinstance(w, torch.Tensor) and w.dtype == torch.uint8 and w.dim() == 2:
            if tuple(w.shape) != (self.out_features, self.in_features // 2):
                error_msgs.append(f"{key}: CPU-layout int4 weight must be [{self.out_features}, {self.in_features // 2}], "
                                  f"got {list(w.shape)}")
            elif self.out_features % 16 != 0:
                error_msgs.append(f"{key}: the CPU layout needs out_features % 16 == 0")
            elif not self.weight.is_cuda:
                error_msgs.append(f"{key}: move the module to the GPU before loading a CPU-layout weight (the converter is a GPU kernel)")
            else:
                if self.cpu_pack_layout is None:
                    warnings.warn(f"{key}: CPU-layout int4 weight with cpu_pack_layout unset: assuming the AVX-512 pack (64, True); "
                                  "set cpu_pack_layout = (32, True) for an AVX2 pack, (32, False) for the plain tier", stacklevel=2)
                block_cols, half_split = self.cpu_pack_layout or (64, True)
                state_dict = dict(state_dict)
                state_dict[key] = ops.int4pack_cpu_to_device(w.to(self.weight.device), block_cols=block_cols, half_split=half_split)
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs)

    @classmethod
    def from_float(cls, linear: nn.Linear, groupsize: int = 128) -> "WeightOnlyInt4Linear":
        if linear.bias is not None and linear.bias.dim() != 1:
            raise ValueError("int4 weight-only requires a 1-D bias or no bias")
        w = linear.weight.detach()
        packed, scale_zero = _pack_int4_weight(w, groupsize)
        mod = cls(linear.in_features, linear.out_features, groupsize=groupsize, bias=linear.bias is not None,
                  device=w.device, dtype=w.dtype)
        mod.weight = packed
        mod.scales_and_zeros = scale_zero
        if linear.bias is not None:
            mod.bias = linear.bias.detach()
        return mod


@register_quantize_module_handler(Int4WeightOnlyConfig)
def _int4_weight_only_transform(module, config):
    """Replace an ``nn.Linear`` with a packed int4 weight-only linear (reference :198-201)."""
    return WeightOnlyInt4Linear.from_float(module, config.groupsize)
