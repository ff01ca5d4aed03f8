"""Module-swap entry point (reference: tensorplay/ao/quantization/quantize_api.py:14-85).

``quantize_(model, config)`` walks ``named_modules()`` and replaces every module the filter accepts
(``nn.Linear`` by default) with what the handler registered for ``type(config)`` returns.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import torch.nn as nn

_HANDLERS: Dict[type, Callable] = {}


def register_quantize_module_handler(config_type: type):
    def deco(fn):
        _HANDLERS[config_type] = fn
        return fn

    return deco


def _is_linear(module: nn.Module, fqn: str) -> bool:
    return isinstance(module, nn.Linear)


def quantize_(model: nn.Module, config, filter_fn: Optional[Callable[[nn.Module, str], bool]] = None) -> nn.Module:
    handler = _HANDLERS.get(type(config))
    if handler is None:
        raise ValueError(f"quantize_: no handler registered for {type(config).__name__}")
    accept = filter_fn or _is_linear
    if accept(model, ""):
        return handler(model, config)
    for fqn, module in list(model.named_modules()):
        for name, child in list(module.named_children()):
            child_fqn = f"{fqn}.{name}" if fqn else name
            if accept(child, child_fqn):
                setattr(module, name, handler(child, config))
    return model
