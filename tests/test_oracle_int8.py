"""Pins for the oracle's integer product, rescale, PackedWeight special case and the
dynamic int8 linear composition (A3, A4, A5, A12).

Independent evidence: the widened numpy product and torch._int_mm on CPU
(reference: test/test_missing_native_ops.py:684-729), the float32 closed form
of the rescale (p10/include/QuantNativeImpl.h:1258-1259), the int64 closed form
of the packed linear (test/quantization/test_packed_quantization.py:54-62) and
manual_int8mp_linear (test/quantization/test_int8_mixed_precision.py:26-34).
"""
import numpy as np
import pytest
import torch

import oracle
from helpers import cast_bits, from_bits


@pytest.mark.parametrize("shape", [(5, 7, 3), (1, 1, 1), (16, 1024, 1024), (64, 12, 32), (33, 257, 65)])
@pytest.mark.parametrize("unsigned", [False, True])
def test_int_mm_matches_widened_product(shape, unsigned):
    M, K, N = shape
    rng = np.random.default_rng(M * 131 + K * 17 + N)
    a = rng.integers(0 if unsigned else -128, 256 if unsigned else 128, size=(M, K)).astype(np.uint8 if unsigned else np.int8)
    a[rng.random(a.shape) < 0.1] = 0  # the reference skips zero entries of A
    b = rng.integers(-128, 128, size=(K, N)).astype(np.int8)
    want = a.astype(np.int32) @ b.astype(np.int32)
    np.testing.assert_array_equal(oracle.int_mm(a, b), want)
    # transposed view of an [N,K] weight, the layout the Python callers pass
    w = np.ascontiguousarray(b.T)
    np.testing.assert_array_equal(oracle.int_mm(a, w.T), want)
    if not unsigned:
        np.testing.assert_array_equal(oracle.int_mm_nk(a, w), want)


def test_int_mm_matches_torch_cpu_library():
    torch.manual_seed(0)
    a = torch.randint(-128, 128, (32, 64), dtype=torch.int8)
    b = torch.randint(-128, 128, (64, 16), dtype=torch.int8)
    np.testing.assert_array_equal(oracle.int_mm(a.numpy(), b.numpy()), torch._int_mm(a, b).numpy())


def test_int_mm_extremes_do_not_overflow_int32():
    K = 6912
    a = np.full((2, K), -128, np.int8)
    b = np.full((K, 2), -128, np.int8)
    assert oracle.int_mm(a, b)[0, 0] == 128 * 128 * K


def test_rescale_closed_form_and_order():
    rng = np.random.default_rng(5)
    acc = rng.integers(-2**20, 2**20, size=(37, 53)).astype(np.int32)
    rs = rng.uniform(1e-3, 1e-1, 37).astype(np.float32)
    cs = rng.uniform(1e-4, 1e-2, 53).astype(np.float32)
    got = oracle.int8_mm_rescale(acc, rs, cs)
    want = (acc.astype(np.float32) * rs[:, None]) * cs[None, :]
    np.testing.assert_array_equal(got, want)
    # the other association differs in the last bit somewhere: the order is part of the spec
    other = acc.astype(np.float32) * (rs[:, None] * cs[None, :])
    assert (other != want).any()
    # bf16 / f16 outputs are one RNE rounding of the same fp32 value
    for dt in ("bf16", "f16"):
        np.testing.assert_array_equal(oracle.int8_mm_rescale(acc, rs, cs, out_dtype=dt), cast_bits(want, dt))
    bias = rng.normal(0, 0.01, 53).astype(np.float32)
    np.testing.assert_array_equal(oracle.int8_mm_rescale(acc, rs, cs, bias=bias), want + bias[None, :])


def test_dynamic_int8_linear_matches_reference_manual_formula():
    # config 1 shape: M=16, K=1024, N=1024, fp32, bias ~ N(0, 0.01)
    rng = np.random.default_rng(2026)
    x = rng.normal(0, 1, (16, 1024)).astype(np.float32)
    w = rng.normal(0, 0.02, (1024, 1024)).astype(np.float32)
    b = rng.normal(0, 0.01, 1024).astype(np.float32)
    xq, xs = oracle.quantize_int8_rowwise(x)
    wq, ws = oracle.quantize_int8_rowwise(w)
    acc = oracle.int_mm(xq, wq.T)
    out = oracle.int8_mm_rescale(acc, xs, ws) + b
    # manual_int8mp_linear: float matmul of the codes, then * A_scale * B_scale
    tx, tw = torch.from_numpy(xq), torch.from_numpy(wq)
    ref = (tx.float() @ tw.float().T) * torch.from_numpy(xs)[:, None] * torch.from_numpy(ws)[None, :] + torch.from_numpy(b)
    np.testing.assert_allclose(out, ref.numpy(), rtol=1e-5, atol=1e-6)
    # and it approximates the float linear
    dense = x @ w.T + b
    assert np.abs(out - dense).max() / np.abs(dense).max() < 2e-2


@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("K", [23, 64])
def test_packed_linear_matches_int64_closed_form(unsigned, K):
    rng = np.random.default_rng(23)
    rows, N = 5, 7
    xcodes = rng.integers(0 if unsigned else -128, 256 if unsigned else 128, size=(rows, K))
    wcodes = rng.integers(-128, 128, size=(N, K))
    xs, xz = 0.021, (137 if unsigned else -13)
    scales = np.linspace(0.007, 0.04, N, dtype=np.float32)
    zps = np.arange(-3, 4, dtype=np.int64)
    bias = np.linspace(-0.7, 0.7, N, dtype=np.float32)
    packed, offsets = oracle.weight_prepack(wcodes.astype(np.int8))
    assert packed.shape == (N, (K + 31) // 32 * 32)
    np.testing.assert_array_equal(offsets, wcodes.sum(1))
    np.testing.assert_array_equal(packed[:, :K], wcodes)
    assert not packed[:, K:].any()
    got = oracle.packed_run_linear_float(xcodes.astype(np.uint8 if unsigned else np.int8), xs, xz, packed, offsets, scales, zps, bias, K)
    acc = (xcodes.astype(np.int64) - xz) @ (wcodes.astype(np.int64) - zps[:, None]).T
    want = acc * xs * scales + bias
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-6)
    # the hot path's special case is the plain integer dot product as float
    plain = oracle.packed_run_linear_float(xcodes.astype(np.uint8 if unsigned else np.int8), 1.0, 0, packed, offsets,
                                           np.ones(N, np.float32), np.zeros(N, np.int64), None, K)
    np.testing.assert_array_equal(plain, (xcodes.astype(np.int64) @ wcodes.astype(np.int64).T).astype(np.float32))
