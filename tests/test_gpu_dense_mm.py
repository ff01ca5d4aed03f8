"""GPU parity: tpq_dense_mm, the plain 16-bit GEMM behind the dequantise-then-multiply routes (reference:
p10/src/backend/cuda/QuantGemmKernels.cu:1339, a vendor GEMM with float32 accumulation).

The reference fixes no summation order, so the check is against the exact product of the same 16-bit inputs in float64:
each output within one unit of the output type plus the drift of a float32 sum of K terms over the sum of |x w|.
Integer-valued inputs whose products and sums are exact in float32 must come out exact.
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import DEV, cast_bits, dev, host

pytestmark = pytest.mark.gpu

ULP = {"f16": 2.0 ** -10, "bf16": 2.0 ** -7}


@pytest.fixture(scope="module")
def ops():
    from tensorplay_amd import ops as _ops

    return _ops


def _run(ops, xb, wb, dtype):
    x, w = dev(xb, dtype), dev(wb, dtype)
    out = torch.full((x.shape[0], w.shape[0]), float("nan"), dtype=x.dtype, device=DEV)
    got = ops._dense_mm(x, w, out)
    assert got is out
    return oracle.to_f32(host(out), dtype).astype(np.float64)


# M, N, K: one and several tiles of 256 and of 128 rows, ragged edges in M and N, N that forbids 16-byte stores, one to
# many stages (a stage is 64 elements of k), more tiles than compute units
SHAPES = [(1, 8, 64), (1, 128, 128), (7, 5, 192), (128, 128, 64), (129, 136, 320), (256, 128, 64), (300, 200, 192), (257, 137, 448),
          (513, 264, 4096), (2048, 1000, 1024), (384, 11008, 256), (1100, 4104, 512), (40, 72, 11008)]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES)
def test_dense_mm_against_the_exact_product(ops, dtype, shape):
    M, N, K = shape
    rng = np.random.default_rng(M * 7919 + N * 31 + K)
    xb = cast_bits(rng.normal(0, 1, (M, K)).astype(np.float32), dtype)
    wb = cast_bits(rng.normal(0, 0.05, (N, K)).astype(np.float32), dtype)
    x64, w64 = oracle.to_f32(xb, dtype).astype(np.float64), oracle.to_f32(wb, dtype).astype(np.float64)
    want = x64 @ w64.T
    mass = np.abs(x64) @ np.abs(w64).T
    got = _run(ops, xb, wb, dtype)
    assert not np.isnan(got).any(), "an output was not written"
    bound = 0.51 * ULP[dtype] * np.abs(want) + K * 2.0 ** -24 * mass + (2.0 ** -24 if dtype == "f16" else 1e-30)
    bad = np.abs(got - want) > bound
    assert not bad.any(), f"{bad.sum()} of {bad.size} outside the bound; worst {np.abs(got - want).max():.3e}"


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("shape", [(300, 200, 192), (256, 136, 640), (77, 1000, 128)])
def test_dense_mm_exact_on_small_integers(ops, dtype, shape):
    """Inputs in -4..4: every product and partial sum is an integer below 2^24, the result below 2^8 in magnitude is
    exact in both output types whatever the order of the sum."""
    M, N, K = shape
    rng = np.random.default_rng(K + M)
    x = rng.integers(-4, 5, (M, K)).astype(np.float32)
    w = (rng.integers(-4, 5, (N, K)) * (rng.random((N, K)) < 0.05)).astype(np.float32)   # sparse: sums stay small
    want = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(want).max() < 256
    got = _run(ops, cast_bits(x, dtype), cast_bits(w, dtype), dtype)
    np.testing.assert_array_equal(got, want)


def test_dense_mm_refuses_what_it_does_not_build(ops):
    from tensorplay_amd import _lib

    lib = _lib.load()
    x = torch.zeros((4, 96), dtype=torch.float16, device=DEV)
    w = torch.zeros((8, 96), dtype=torch.float16, device=DEV)
    out = torch.full((4, 8), 3.0, dtype=torch.float16, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    assert lib.tpq_dense_mm(x.data_ptr(), ops._DT[torch.float16], 4, 96, w.data_ptr(), 8, out.data_ptr(), s) == _lib.TPQ_ERR_UNSUPPORTED
    assert lib.tpq_dense_mm(x.data_ptr(), ops._DT[torch.float32], 4, 48, w.data_ptr(), 8, out.data_ptr(), s) == _lib.TPQ_ERR_UNSUPPORTED   # float32: multiples of 32
    assert lib.tpq_dense_mm(x.data_ptr(), 7, 4, 64, w.data_ptr(), 8, out.data_ptr(), s) == _lib.TPQ_ERR_UNSUPPORTED
    assert lib.tpq_dense_mm(x.data_ptr(), ops._DT[torch.float16], 0, 64, w.data_ptr(), 8, out.data_ptr(), s) == 0
    torch.cuda.synchronize()
    assert bool((out == 3.0).all())
    # the wrapper falls back to the framework's GEMM for such K
    xr = torch.randn((4, 96), dtype=torch.float16, device=DEV)
    wr = torch.randn((8, 96), dtype=torch.float16, device=DEV)
    got = ops._dense_mm(xr, wr, torch.empty((4, 8), dtype=torch.float16, device=DEV))
    torch.testing.assert_close(got.float(), xr.float() @ wr.float().t(), rtol=2e-3, atol=2e-2)


@pytest.mark.parametrize("shape", [(1, 8, 32), (7, 5, 96), (129, 136, 320), (300, 200, 192), (257, 137, 448), (513, 264, 4096),
                                   (2048, 1000, 1024), (384, 11008, 256), (40, 72, 11008)])
def test_dense_mm_float32(shape):
    """float32 operands (a stage is 32 elements of k, four v_mfma_f32_16x16x4_f32 per fragment): against the exact
    product in float64, every output within the drift of a float32 sum of K terms; small integers exact."""
    from tensorplay_amd import _lib
    lib = _lib.load()
    M, N, K = shape
    rng = np.random.default_rng(M * 7919 + N * 31 + K + 1)
    for ints in (False, True):
        if ints:
            x = rng.integers(-8, 9, (M, K)).astype(np.float32)
            w = rng.integers(-8, 9, (N, K)).astype(np.float32)
        else:
            x = rng.normal(0, 1, (M, K)).astype(np.float32)
            w = rng.normal(0, 0.05, (N, K)).astype(np.float32)
        xd, wd = torch.from_numpy(x).to(DEV), torch.from_numpy(w).to(DEV)
        out = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
        rc = lib.tpq_dense_mm(xd.data_ptr(), _lib.F32, M, K, wd.data_ptr(), N, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
        assert rc == 0, _lib.last_error()
        got = out.cpu().numpy().astype(np.float64)
        want = x.astype(np.float64) @ w.astype(np.float64).T
        assert not np.isnan(got).any(), "an output was not written"
        if ints:
            np.testing.assert_array_equal(got, want)
        else:
            mass = np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64).T
            bad = np.abs(got - want) > (K + 2) * 2.0 ** -24 * mass + 1e-30
            assert not bad.any(), f"{bad.sum()} of {bad.size} outside the bound; worst {np.abs(got - want).max():.3e}"
