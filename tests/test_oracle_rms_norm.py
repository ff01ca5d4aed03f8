"""Pins for the oracle's rms_norm (reference: p10/src/backend/cpu/NormalizationKernels.cpp:1355-1453,
tensorplay/nn/functional.py:2350-2372): PyTorch's own CPU rms_norm as the library twin, the float64 closed form,
and what the definition fixes (scaling by a power of two at eps = 0, constant rows, zero rows)."""
import numpy as np
import pytest
import torch

import oracle
from helpers import TORCH_DT, bits_of, cast_bits, from_bits

ULP = {"f32": 2.0 ** -23, "f16": 2.0 ** -10, "bf16": 2.0 ** -7}


def _as_f32(a, dtype):
    return a if dtype == "f32" else oracle.to_f32(a, dtype)


def _inputs(rng, shape, dtype, offset=0.3, spread=2.0):
    x = (rng.normal(size=shape) * spread + offset).astype(np.float32)
    w = rng.uniform(0.5, 1.5, shape[1]).astype(np.float32)
    if dtype == "f32":
        return x, w
    return cast_bits(x, dtype), cast_bits(w, dtype)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(1, 1), (3, 7), (16, 1024), (5, 4096), (2, 11008)])
def test_against_torch_cpu_and_float64(dtype, shape):
    rng = np.random.default_rng(shape[0] * 131 + shape[1])
    x, w = _inputs(rng, shape, dtype)
    got, y64 = oracle.rms_norm(x, dtype, w, 1e-5, want_f64=True)
    xt = torch.from_numpy(x) if dtype == "f32" else from_bits(x, dtype)
    wt = torch.from_numpy(w) if dtype == "f32" else from_bits(w, dtype)
    twin = torch.nn.functional.rms_norm(xt, (shape[1],), wt, 1e-5).float().numpy()
    g = _as_f32(got, dtype).astype(np.float64)
    # the library twin adds the squares in another order (the serial float32 sum of the reference drifts by about
    # sqrt(K) half-units) and may round x * inv * w differently by one unit; float16 results below 2^-14 are subnormal
    drift = np.sqrt(shape[1]) * 2.0 ** -24
    floor = 2.0 ** -24 if dtype == "f16" else 1e-30
    assert np.all(np.abs(g - twin) <= (2.5 * ULP[dtype] + drift) * np.abs(twin) + floor)
    # closed form in float64 on the same inputs: one rounding of the output type plus the float32 steps
    xf, wf = _as_f32(x, dtype).astype(np.float64), _as_f32(w, dtype).astype(np.float64)
    closed = xf / np.sqrt((xf ** 2).mean(-1, keepdims=True) + np.float64(np.float32(1e-5))) * wf
    np.testing.assert_allclose(y64, closed, rtol=1e-12, atol=0)
    assert np.all(np.abs(g - closed) <= (0.5 * ULP[dtype] + 4 * 2.0 ** -23 + drift) * np.abs(closed) * 1.01 + floor)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_scaling_by_a_power_of_two_changes_nothing_at_eps_zero(dtype):
    rng = np.random.default_rng(11)
    x, w = _inputs(rng, (6, 520), dtype)
    base = oracle.rms_norm(x, dtype, w, 0.0)
    for p in (1, 2, 5):  # up only: exact in every type (no overflow), while scaling down could make float16 inputs subnormal
        xs = _as_f32(x, dtype) * np.float32(2.0 ** p)
        xs = xs if dtype == "f32" else cast_bits(xs, dtype)
        np.testing.assert_array_equal(oracle.rms_norm(xs, dtype, w, 0.0), base)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_constant_and_zero_rows(dtype):
    k = 256
    x = np.zeros((3, k), np.float32)
    x[0] = 3.0        # mean of squares 9: inv = 1/3 up to rounding, out = w up to two float32 roundings
    x[1] = -0.5
    w = np.linspace(0.5, 1.5, k).astype(np.float32)
    xb, wb = (x, w) if dtype == "f32" else (cast_bits(x, dtype), cast_bits(w, dtype))
    got = _as_f32(oracle.rms_norm(xb, dtype, wb, 0.0), dtype)
    wv = _as_f32(wb, dtype)
    tol = ULP[dtype] + 3 * 2.0 ** -23
    np.testing.assert_allclose(got[0], wv, rtol=tol, atol=0)
    np.testing.assert_allclose(got[1], -wv, rtol=tol, atol=0)
    zero = _as_f32(oracle.rms_norm(xb[2:], dtype, wb, 1e-5), dtype)
    np.testing.assert_array_equal(zero, np.zeros((1, k), np.float32))
    # without a weight the result is x * inv alone
    plain = _as_f32(oracle.rms_norm(xb[:1], dtype, None, 0.0), dtype)
    np.testing.assert_allclose(plain, np.ones((1, k), np.float32), rtol=tol, atol=0)


def test_dropped_term_or_wrong_order_would_show():
    """eps inside the square root (not added to the root), the mean (not the sum) of the squares, weight applied after
    the normalization: each of these mistakes moves the result by far more than the tolerances above."""
    rng = np.random.default_rng(3)
    x = (rng.normal(size=(2, 64)) * 0.01).astype(np.float32)   # small values: eps = 1e-2 matters
    w = rng.uniform(0.5, 1.5, 64).astype(np.float32)
    got = oracle.rms_norm(x, "f32", w, 1e-2).astype(np.float64)
    xf = x.astype(np.float64)
    right = xf / np.sqrt((xf ** 2).mean(-1, keepdims=True) + np.float64(np.float32(1e-2))) * w
    wrong_eps = xf / (np.sqrt((xf ** 2).mean(-1, keepdims=True)) + 1e-2) * w
    wrong_sum = xf / np.sqrt((xf ** 2).sum(-1, keepdims=True) + 1e-2) * w
    np.testing.assert_allclose(got, right, rtol=1e-6)
    assert np.abs(got - wrong_eps).max() > 1e-3 * np.abs(right).max()
    assert np.abs(got - wrong_sum).max() > 1e-3 * np.abs(right).max()
