"""BitNet b1.58 host code (reference: tensorplay/ao/quantization/bitnet.py:48-136, 215-241, 528-547).

The reference unpacks the 2-bit weight to int8 on every forward, multiplies through its packed int8
linear and applies two elementwise scales; here the packed weight goes straight into one kernel
that produces ``(float(acc) * row_scale) * scale (+ bias)``, the same fp32 operations in the same
order.
"""
from __future__ import annotations

from typing import Optional, Tuple, Union

import torch
import torch.nn as nn

from ... import ops

pack_ternary = ops.pack_ternary
unpack_ternary = ops.unpack_ternary


def get_bitnet_scale(weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """mean(|W|) clamped at eps, in the weight's dtype (reference :48-55)."""
    return weight.abs().mean().clamp(min=eps)


def quantize_bitnet_weight(weight: torch.Tensor, scale: Optional[torch.Tensor] = None,
                           eps: float = 1e-5) -> Tuple[torch.Tensor, torch.Tensor]:
    """codes = clamp(round(W.float() / scale), -1, 1) as int8, and the scale (reference :58-69)."""
    scale = get_bitnet_scale(weight, eps) if scale is None else scale.clamp(min=eps)
    codes = (weight.float() / scale).round().clamp(-1, 1).to(torch.int8)
    return codes, scale


def quantize_int8_rowwise(input: torch.Tensor, eps: float = 1e-5) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row symmetric int8 codes and float32 scales [.., 1] (reference :110-136, device branch)."""
    lead = input.shape[:-1]
    codes, scales = ops._quantize_int8_rowwise(input.reshape(-1, input.shape[-1]), eps)
    return codes.reshape(*lead, input.shape[-1]), scales.reshape(*lead, 1)


def bitnet_linear_packed(input: torch.Tensor, packed: torch.Tensor, scale: Union[torch.Tensor, float],
                         in_features: int, bias: Optional[torch.Tensor] = None, eps: float = 1e-5) -> torch.Tensor:
    """BitNet linear from pre-packed ternary weights (reference :215-241): float32 output
    ``(float(x_i8 . codes) * row_scale) * scale (+ bias)``.  A tensor ``scale`` is read back to the
    host once per call; modules keep it as a Python float instead."""
    batch_dims = input.shape[:-1]
    x = input.reshape(-1, in_features)
    x_i8, row_scale = ops._quantize_int8_rowwise(x, eps)
    w_scale = float(scale)
    out = ops.ternary_mm(x_i8, row_scale, packed, w_scale, in_features, bias=bias, out_dtype=torch.float32)
    return out.reshape(*batch_dims, packed.shape[0])


class BitNetPacked2bitLinear(nn.Module):
    """Inference module over a 2-bit packed ternary weight (reference _BitNetPacked2bitLinear :528-547).

    State: ``int_data`` (uint8 [N, ceil(K/4)]) and ``scale`` (0-dim, the weight's dtype), the two inner tensors the
    reference's packed weight subclass flattens to (``BitNetPacked2bitLinearWeight.__tensor_flatten__``, :478-486),
    plus ``bias``.  load_state_dict also takes ``weight`` holding such a subclass instance (anything with
    ``int_data`` and ``scale`` attributes) or a dict of the two, which is what a reference model's ``weight`` entry is."""

    def __init__(self, packed: torch.Tensor, scale: Union[torch.Tensor, float], in_features: int,
                 bias: Optional[torch.Tensor] = None, eps: float = 1e-5):
        super().__init__()
        self.in_features = in_features
        self.out_features = packed.shape[0]
        self.eps = eps
        self.register_buffer("int_data", packed)
        scale_t = scale.detach().reshape(()) if isinstance(scale, torch.Tensor) else torch.tensor(float(scale), dtype=torch.float32)
        self.register_buffer("scale", scale_t.to(packed.device))
        self._scale_value = float(scale_t)   # host copy: the kernel takes the scale by value, no sync per forward
        if bias is not None:
            self.register_buffer("bias", bias)
        else:
            self.bias = None

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        wkey = prefix + "weight"
        if wkey in state_dict:   # the reference's flattened subclass: weight -> (int_data, scale)
            w = state_dict[wkey]
            inner = w if isinstance(w, dict) else {"int_data": getattr(w, "int_data", None), "scale": getattr(w, "scale", None)}
            if isinstance(inner.get("int_data"), torch.Tensor) and isinstance(inner.get("scale"), torch.Tensor):
                state_dict = {k: v for k, v in state_dict.items() if k != wkey}
                state_dict[prefix + "int_data"] = inner["int_data"]
                state_dict[prefix + "scale"] = inner["scale"].reshape(())
            else:
                error_msgs.append(f"{wkey}: expected a packed BitNet weight with int_data and scale")
        skey = prefix + "scale"
        if isinstance(state_dict.get(skey), torch.Tensor) and state_dict[skey].numel() == 1:
            state_dict = dict(state_dict)
            state_dict[skey] = state_dict[skey].reshape(())
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs)
        self._scale_value = float(self.scale)

    def _apply(self, fn, recurse=True):
        super()._apply(fn, recurse)
        self._scale_value = None   # a dtype change rounds the scale: read again at the next forward (no copy here: meta tensors, no sync per .to())
        return self

    @classmethod
    def from_float(cls, linear: nn.Linear, eps: float = 1e-5) -> "BitNetPacked2bitLinear":
        codes, scale = quantize_bitnet_weight(linear.weight.detach(), eps=eps)
        bias = None if linear.bias is None else linear.bias.detach()
        return cls(pack_ternary(codes), scale, linear.in_features, bias, eps)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if self._scale_value is None:
            self._scale_value = float(self.scale)
        return bitnet_linear_packed(input, self.int_data, self._scale_value, self.in_features, self.bias, self.eps)
