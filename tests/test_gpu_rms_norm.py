"""GPU parity: tpq_rms_norm against the CPU oracle (reference: p10/src/backend/cpu/NormalizationKernels.cpp:1355-1453).

Floating point: the kernel adds the squares of a row in a tree, the reference's CPU kernel serially, so inv may differ
in its last bits; the bound is one unit of the output type plus the drift of a float32 sum of K terms (stated below).
Scaling a row by a power of two at eps = 0 must not change a single bit, on the device as in the oracle.
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import DEV, cast_bits, dev, host

pytestmark = pytest.mark.gpu

ULP = {"f32": 2.0 ** -23, "f16": 2.0 ** -10, "bf16": 2.0 ** -7}


@pytest.fixture(scope="module")
def ops():
    from tensorplay_amd import ops as _ops

    return _ops


def _f32(a, dtype):
    return a if dtype == "f32" else oracle.to_f32(a, dtype)


def _check(got_bits, want_bits, dtype, k):
    got, want = _f32(got_bits, dtype).astype(np.float64), _f32(want_bits, dtype).astype(np.float64)
    tol = 1.01 * ULP[dtype] + 2 * np.sqrt(k) * 2.0 ** -24   # one unit of the output type + the drift of the two float32 sums
    floor = 2.0 ** -24 if dtype == "f16" else 1e-30          # float16 subnormals
    bad = np.abs(got - want) > tol * np.abs(want) + floor
    assert not bad.any(), f"{bad.sum()} of {bad.size} outside {tol:.2e} relative; worst {np.abs(got - want).max():.3e}"
    # and most elements are identical: a wrong formula would not hide inside the bound
    if dtype != "f32":  # (float32: a last-bit difference in inv shows in about half of the row)
        assert (got_bits == want_bits).mean() > 0.97


SHAPES = [(1, 1), (3, 5), (8, 4096), (5, 100), (4, 24), (7, 2560), (2, 6912), (3, 11008), (2, 16384), (1, 32768), (2, 20000),
          (300, 2048), (2048, 4096), (64, 8200), (33, 136)]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES)
def test_rms_norm_against_oracle(ops, dtype, shape):
    rng = np.random.default_rng(shape[0] * 977 + shape[1])
    x = (rng.normal(size=shape) * 2.0 + 0.3).astype(np.float32)
    w = rng.uniform(0.5, 1.5, shape[1]).astype(np.float32)
    xb, wb = (x, w) if dtype == "f32" else (cast_bits(x, dtype), cast_bits(w, dtype))
    want = oracle.rms_norm(xb, dtype, wb, 1e-5)
    got = host(ops.rms_norm(dev(xb, dtype), dev(wb, dtype), 1e-5))
    _check(got, want, dtype, shape[1])
    # without a weight
    got = host(ops.rms_norm(dev(xb, dtype), None, 1e-6))
    _check(got, oracle.rms_norm(xb, dtype, None, 1e-6), dtype, shape[1])


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("k", [520, 4096, 100, 40000])
def test_power_of_two_scaling_is_exact_at_eps_zero(ops, dtype, k):
    rng = np.random.default_rng(k)
    x = (rng.normal(size=(4, k)) + 0.1).astype(np.float32)
    w = rng.uniform(0.5, 1.5, k).astype(np.float32)
    xb, wb = (x, w) if dtype == "f32" else (cast_bits(x, dtype), cast_bits(w, dtype))
    base = host(ops.rms_norm(dev(xb, dtype), dev(wb, dtype), 0.0))
    for p in (1, 3):  # up only: scaling down would push the smallest float16 inputs into the subnormal range
        xs = _f32(xb, dtype) * np.float32(2.0 ** p)
        xs = xs if dtype == "f32" else cast_bits(xs, dtype)
        np.testing.assert_array_equal(host(ops.rms_norm(dev(xs, dtype), dev(wb, dtype), 0.0)), base)


def test_leading_dimensions_views_and_errors(ops):
    x = torch.randn(2, 3, 256, device=DEV, dtype=torch.float16)
    w = torch.rand(256, device=DEV, dtype=torch.float16) + 0.5
    y = ops.rms_norm(x, w, 1e-5)
    assert y.shape == x.shape and y.dtype == x.dtype
    assert torch.equal(y.reshape(6, 256), ops.rms_norm(x.reshape(6, 256), w, 1e-5))
    # a strided view is read through a packed copy, like the reference's input.contiguous()
    xt = torch.randn(256, 6, device=DEV, dtype=torch.float16).t()
    assert torch.equal(ops.rms_norm(xt, w, 1e-5), ops.rms_norm(xt.contiguous(), w, 1e-5))
    assert ops.rms_norm(torch.empty(0, 256, device=DEV, dtype=torch.float16), w).shape == (0, 256)
    with pytest.raises(ValueError):
        ops.rms_norm(x, w[:100], 1e-5)
    with pytest.raises(TypeError):
        ops.rms_norm(x.to(torch.int32), None, 1e-5)
    with pytest.raises(RuntimeError):
        ops.rms_norm(x.cpu(), None, 1e-5)


def test_prefill_block_full_size_properties(ops):
    """2048 x 4096 bf16: every row has unit mean square after the norm (weight None), to the rounding of the type."""
    x = (torch.randn(2048, 4096, device=DEV) * 3.0).to(torch.bfloat16)
    y = ops.rms_norm(x, None, 1e-6).float()
    ms = (y * y).mean(-1)
    assert torch.all((ms - 1.0).abs() < 2e-3)
    assert torch.equal(torch.sign(y), torch.sign(x.float()))
