"""Host-side logic of the ao mirror that needs no GPU: the weight quantizers' closed forms, the
module-swap registry, argument validation, and the loud failure when tensors are not on the GPU."""
import numpy as np
import pytest
import torch
import torch.nn as nn

from tensorplay_amd.ao.quantization import (Int4WeightOnlyConfig, WeightOnlyInt4Linear, _quantize_int4_groupwise,
                                            get_bitnet_scale, quantize_, quantize_bitnet_weight)
from tensorplay_amd.ao.quantization import quantize_api


def test_int4_groupwise_closed_form():
    """reference int4_weight_only.py:62-82: symmetric, scale = max|w|/8, code = round(w/s) in [-8,7], +8."""
    rng = np.random.default_rng(5)
    w = rng.normal(0, 0.02, (24, 256)).astype(np.float32)
    codes, scale, zero = _quantize_int4_groupwise(torch.from_numpy(w), 64)
    wg = w.reshape(24, 4, 64)
    s = np.maximum(np.abs(wg).max(-1) / np.float32(8.0), np.float32(1e-8))
    want = (np.clip(np.rint(wg / s[..., None]), -8, 7) + 8).astype(np.int32).reshape(24, 256)
    np.testing.assert_array_equal(codes.numpy(), want)
    np.testing.assert_array_equal(scale.numpy(), s)
    assert codes.dtype == torch.int32 and not zero.any()
    assert codes.min() >= 0 and codes.max() <= 15
    with pytest.raises(ValueError):
        _quantize_int4_groupwise(torch.zeros(8, 100), 64)


def test_bitnet_weight_quantizer_literal():
    """reference test_native_1bit.py:213-224."""
    w = torch.tensor([[.4, -.1, .2, -.3], [.0, .6, -.8, .1]], dtype=torch.float32)
    scale = get_bitnet_scale(w)
    np.testing.assert_allclose(scale.item(), np.abs(w.numpy()).mean(), rtol=1e-6)
    codes, scale2 = quantize_bitnet_weight(w, scale)
    assert codes.dtype == torch.int8
    np.testing.assert_array_equal(codes.numpy(), np.clip(np.round(w.numpy() / scale.item()), -1, 1))
    assert get_bitnet_scale(torch.zeros(4, 4)).item() == pytest.approx(1e-5)


def test_quantize_registry():
    class Unknown:
        pass

    with pytest.raises(ValueError):
        quantize_(nn.Linear(32, 8), Unknown())
    seen = []

    class Cfg:
        pass

    @quantize_api.register_quantize_module_handler(Cfg)
    def _h(module, config):
        seen.append(module)
        return nn.Identity()

    model = nn.Sequential(nn.Linear(32, 32), nn.ReLU(), nn.Sequential(nn.Linear(32, 8)))
    quantize_(model, Cfg())
    assert len(seen) == 2 and isinstance(model[0], nn.Identity) and isinstance(model[2][0], nn.Identity)
    assert isinstance(model[1], nn.ReLU)
    assert quantize_api._HANDLERS[Int4WeightOnlyConfig].__name__ == "_int4_weight_only_transform"


def test_module_shapes_and_validation():
    m = WeightOnlyInt4Linear(256, 64, groupsize=128)
    assert m.weight.shape == (8, 8, 32, 1) and m.weight.dtype == torch.int32
    assert m.scales_and_zeros.shape == (2, 64, 2) and m.bias is None
    with pytest.raises(ValueError):
        WeightOnlyInt4Linear(100, 64)
    with pytest.raises(ValueError):
        WeightOnlyInt4Linear(256, 64, groupsize=96)


def test_no_cpu_fallback():
    """CPU tensors are refused: the product has no host path."""
    m = WeightOnlyInt4Linear(256, 64, groupsize=128)
    with pytest.raises((RuntimeError, ValueError, TypeError)):
        m(torch.zeros(1, 256, dtype=torch.float16))
    with pytest.raises((RuntimeError, ValueError, TypeError)):
        WeightOnlyInt4Linear.from_float(nn.Linear(256, 64, bias=False))


def test_fused_int4_ops_check_the_packed_extent_on_the_host():
    """add / swiglu / multi validate layout, K extent and group size before any launch: the kernels only receive
    pointers, so a packed weight that covers fewer k than the activations must never reach them.  CPU tensors
    are enough: every check below fires before the device check."""
    from tensorplay_amd import ops

    x = torch.zeros(2, 256, dtype=torch.float16)
    good = torch.zeros(4, 8, 32, 1, dtype=torch.int32)       # N = 32, K = 256
    narrow = torch.zeros(4, 4, 32, 1, dtype=torch.int32)     # covers K = 128 only
    sz = torch.zeros(2, 32, 2, dtype=torch.float16)
    res = torch.zeros(2, 32, dtype=torch.float16)
    for call in (lambda w, s, g: ops.int4pack_mm_add(x, w, g, s, res),
                 lambda w, s, g: ops.int4pack_mm_swiglu(x, w, good, g, s, sz),
                 lambda w, s, g: ops.int4pack_mm_swiglu(x, good, w, g, sz, s),    # the up weight is checked too
                 lambda w, s, g: ops.int4pack_mm_multi(x, [good, w], g, [sz, s])):
        with pytest.raises(ValueError, match="K dimension does not match"):
            call(narrow, sz, 128)
        with pytest.raises(ValueError, match="qGroupSize"):
            call(good, sz, 96)
        with pytest.raises(ValueError, match="qScaleAndZeros"):
            call(good, torch.zeros(1, 32, 2, dtype=torch.float16), 128)
        with pytest.raises(ValueError, match="layout is invalid"):
            call(torch.zeros(4, 1, 32, 8, dtype=torch.int32), sz, 128)   # innerKTiles = 16
        with pytest.raises(TypeError):
            call(torch.zeros(4, 8, 16, 1, dtype=torch.int32), sz, 128)
    # with consistent operands the only thing left to fail on the host is the missing GPU
    with pytest.raises(RuntimeError):
        ops.int4pack_mm_add(x, good, 128, sz, res)


def test_bitnet_packed_linear_moves_without_reading_its_scale():
    """.to() / .half() of a model must not copy the scale to the host (a device sync per call, an error on meta
    tensors): the cached value is dropped and read again at the next forward."""
    from tensorplay_amd.ao.quantization import BitNetPacked2bitLinear

    mod = BitNetPacked2bitLinear(torch.zeros(8, 4, dtype=torch.uint8), 0.5, 16, bias=torch.zeros(8))
    assert mod._scale_value == 0.5
    mod.half()
    assert mod._scale_value is None
    mod.to("meta")   # raised before: float() of a meta tensor
    assert mod.scale.is_meta and mod._scale_value is None
