"""GPU parity: fused row-wise quantizer vs the CPU oracle, bit-exact codes and scales."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import DEV, cast_bits, dev, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from tensorplay_amd import ops as _ops

    return _ops


SHAPES = [(1, 1), (3, 5), (16, 1024), (7, 2560), (1, 6912), (5, 4099), (4, 8), (2, 16384), (2, 20000),
          (3, 16392), (128, 6912), (300, 2048), (2048, 4096),
          (1000, 64), (77, 56), (33, 128), (5, 200), (129, 512), (9, 264), (70, 1000), (4097, 1024), (3, 1032),
          (3, 28672), (2, 65536), (2, 65544), (5, 40000)]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES)
def test_int8_rowwise_bit_exact(ops, dtype, shape):
    rng = np.random.default_rng(shape[0] * 7919 + shape[1])
    x = rng.normal(size=shape).astype(np.float32)
    if shape[0] > 2:
        x[1] = 0.0                       # all-zero row: scale = eps / 127, codes 0
        x[2] *= 1e-7                     # below eps
    if shape == (2048, 4096):            # outlier columns of the prefill configuration
        x[:, rng.choice(4096, 41, replace=False)] *= 20.0
    xb = cast_bits(x, dtype)
    want_codes, want_scales = oracle.quantize_int8_rowwise(xb, dtype, 1e-5)
    codes, scales = ops._quantize_int8_rowwise(dev(xb, dtype), 1e-5)
    assert codes.dtype == torch.int8 and scales.dtype == torch.float32 and scales.shape == (shape[0],)
    np.testing.assert_array_equal(host(scales), want_scales)
    np.testing.assert_array_equal(host(codes), want_codes)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_lowbit_variants_bit_exact(ops, dtype):
    rng = np.random.default_rng(5)
    x = rng.normal(size=(37, 1000)).astype(np.float32)
    x[3, :5] = [0.5, 1.5, 2.5, -0.5, -1.5]
    xb = cast_bits(x, dtype)
    xd = dev(xb, dtype)
    for fn, ofn in ((ops._quantize_int4_rowwise, oracle.quantize_int4_rowwise),
                    (ops._quantize_int2_rowwise, oracle.quantize_int2_rowwise),
                    (ops._quantize_binary_rowwise, oracle.quantize_binary_rowwise)):
        c, s = fn(xd, 1e-8)
        wc, ws = ofn(xb, dtype, 1e-8)
        np.testing.assert_array_equal(host(c), wc)
        np.testing.assert_array_equal(host(s), ws)


def test_ties_round_to_even(ops):
    x = torch.tensor([[127, -127, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5]], device=DEV)
    codes, scales = ops._quantize_int8_rowwise(x, 1e-5)
    assert scales.item() == 1.0
    assert codes.cpu().tolist() == [[127, -127, 0, 2, 2, 0, -2, -2]]


def test_non_contiguous_and_empty_and_errors(ops):
    x = torch.randn(64, 96, device=DEV)
    view = x[:, ::2]
    c, s = ops._quantize_int8_rowwise(view, 1e-5)
    wc, ws = oracle.quantize_int8_rowwise(view.cpu().contiguous().numpy())
    np.testing.assert_array_equal(host(c), wc)
    np.testing.assert_array_equal(host(s), ws)
    c, s = ops._quantize_int8_rowwise(torch.empty(0, 8, device=DEV), 1e-5)
    assert c.shape == (0, 8) and s.shape == (0,)
    with pytest.raises(ValueError):
        ops._quantize_int8_rowwise(torch.zeros(2, 2, 2, device=DEV), 1e-5)
    with pytest.raises(TypeError):
        ops._quantize_int8_rowwise(torch.zeros(2, 2, device=DEV, dtype=torch.float64), 1e-5)
