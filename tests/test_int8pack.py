"""_weight_int8pack_mm: oracle pins (CPU) and HIP parity (GPU).

Reference semantics: p10/src/backend/cuda/QuantGemmKernels.cu:86-180, 339-405; known-answer example
and closed form from test/test_mps.py:1052-1061."""
import numpy as np
import pytest

import oracle
from helpers import cast_bits, rel_err

A_LIT = np.array([[0.5, -1.0, 2.0, 0.25], [1.0, 0.5, -0.5, 2.0]], np.float32)
W_LIT = np.array([[1, -2, 0, 1], [0, 1, -1, 2], [2, 0, 1, -1]], np.int8)
S_LIT = np.array([0.5, 1.0, 2.0], np.float32)


def test_oracle_literal_and_closed_form():
    ref = (A_LIT @ W_LIT.astype(np.float32).T) * S_LIT
    np.testing.assert_allclose(oracle.weight_int8pack_mm(A_LIT, "f32", W_LIT, S_LIT), ref, atol=1e-5)
    rng = np.random.default_rng(8005)
    x = rng.normal(0, 1, (5, 333)).astype(np.float32)
    w = rng.integers(-128, 128, (17, 333), dtype=np.int8)
    s = rng.uniform(0.001, 0.02, 17).astype(np.float32)
    want = (x.astype(np.float64) @ w.astype(np.float64).T) * s
    for dt in ("f32", "f16", "bf16"):
        xb = cast_bits(x, dt)
        got, y64 = oracle.weight_int8pack_mm(xb, dt, w, s, want_f64=True)
        want_dt = (oracle.to_f32(xb, dt).astype(np.float64) @ w.astype(np.float64).T) * s
        np.testing.assert_allclose(y64, want_dt, rtol=1e-12, atol=1e-12)
        assert rel_err(oracle.to_f32(got, dt), want_dt) < {"f32": 1e-5, "f16": 1e-3, "bf16": 1e-2}[dt]
    assert rel_err(oracle.to_f32(oracle.weight_int8pack_mm(x, "f32", w, s), "f32"), want) < 1e-5


CASES = [(1, 4096, 512), (4, 1024, 136), (16, 256, 40), (17, 384, 72), (2, 100, 9), (8, 16, 3), (33, 128, 24), (1, 11008, 256),
         # every shape of workgroup of the decode kernel: 16 / 32 channels, 16 / 32 rows per pass, ragged N
         (32, 256, 8200), (64, 128, 50), (9, 128, 16390), (3, 256, 16400), (24, 384, 10250), (40, 128, 10240),
         # one row through the row kernel: a last turn that is partly past K, several passes per channel, ragged N,
         # the three workgroup sizes (by N K), K of 16 only
         (1, 4112, 10), (1, 16, 7), (1, 28672, 130), (1, 8192, 8200), (1, 4096, 32772), (1, 65536, 12), (1, 48, 1),
         # two rows on the same kernel (K up to 32768; longer rows take the matrix-core kernel)
         (2, 4112, 10), (2, 32, 5), (2, 28672, 130), (2, 8192, 8200), (2, 4096, 32772), (2, 36864, 12),
         # the all-in-flight matrix-core kernel (3..16 rows, K = 2048..14336): 4 / 8 / 16 rows through LDS, every width of
         # workgroup, a dead last step (K = 2048, 5120, 11008), ragged N, more workgroups than one pass
         (3, 2048, 72), (5, 4096, 4104), (8, 4096, 11008), (4, 4096, 16392), (9, 4096, 136), (16, 5120, 264),
         (7, 8192, 136), (8, 11008, 4104), (6, 14336, 264), (13, 11008, 72),
         # ... 17..32 rows as two blocks of 16 rows against the same weight registers (K = 3072..4096): a partial second
         # block, ragged N, every width of workgroup, a slab of 32 plus a rest
         (17, 3072, 72), (32, 4096, 264), (25, 3584, 136), (31, 4096, 8200), (20, 4096, 11008), (50, 4096, 72)]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("M,K,N", CASES)
def test_gpu_matches_oracle(dtype, M, K, N):
    from gpu_util import dev
    from tensorplay_amd import ops

    rng = np.random.default_rng(M * 7919 + K + N)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    w = rng.integers(-128, 128, (N, K), dtype=np.int8)
    s = rng.uniform(0.001, 0.02, N).astype(np.float32)
    xb = cast_bits(x, dtype)
    got = ops._weight_int8pack_mm(dev(xb, dtype), dev(w), dev(s))
    assert got.shape == (M, N)
    _, y64 = oracle.weight_int8pack_mm(xb, dtype, w, s, want_f64=True)
    # fp32 accumulation: 1e-3 of the exact sums for fp32 / fp16 outputs, 1e-2 for bf16 (output rounding)
    assert rel_err(got.float().cpu().numpy(), y64) < {"f32": 1e-5, "f16": 1e-3, "bf16": 1e-2}[dtype]


@pytest.mark.gpu
def test_gpu_literal_and_errors():
    import torch
    from gpu_util import dev, host
    from tensorplay_amd import ops

    ref = (A_LIT @ W_LIT.astype(np.float32).T) * S_LIT
    np.testing.assert_allclose(host(ops._weight_int8pack_mm(dev(A_LIT), dev(W_LIT), dev(S_LIT))), ref, atol=1e-5)
    with pytest.raises(TypeError):
        ops._weight_int8pack_mm(dev(A_LIT), dev(W_LIT.astype(np.int32)), dev(S_LIT))
    with pytest.raises(ValueError):
        ops._weight_int8pack_mm(dev(A_LIT), dev(W_LIT[:, :3].copy()), dev(S_LIT))
    with pytest.raises(ValueError):
        ops._weight_int8pack_mm(dev(A_LIT), dev(W_LIT), dev(S_LIT[:2].copy()))
    assert ops._weight_int8pack_mm(dev(A_LIT[:0]), dev(W_LIT), dev(S_LIT)).shape == (0, 3)


@pytest.mark.gpu
def test_gpu_all_positive_activations_full_width():
    """Offsets cancel exactly: constant-sign activations at K = 11008 keep fp32 accuracy."""
    from gpu_util import dev
    from tensorplay_amd import ops

    rng = np.random.default_rng(99)
    M, K, N = 3, 11008, 64
    x = np.abs(rng.normal(0, 1, (M, K))).astype(np.float32) + 1.0
    w = rng.integers(-128, 128, (N, K), dtype=np.int8)
    s = np.full(N, 0.01, np.float32)
    xb = cast_bits(x, "f16")
    got = ops._weight_int8pack_mm(dev(xb, "f16"), dev(w), dev(s)).float().cpu().numpy()
    _, y64 = oracle.weight_int8pack_mm(xb, "f16", w, s, want_f64=True)
    assert rel_err(got, y64) < 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
def test_gpu_many_rows_take_the_dense_route(dtype):
    """More rows than INT8PACK_PREFILL_ROWS: dense weight T(w * scale) + one dense GEMM, within the same bounds."""
    import torch
    from tensorplay_amd import ops
    rng = np.random.default_rng(77)
    M, K, N = ops.INT8PACK_PREFILL_ROWS + 9, 272, 40
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = rng.integers(-128, 128, (N, K)).astype(np.int8)
    s = rng.uniform(0.001, 0.02, N).astype(np.float32)
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[dtype]
    xt = torch.from_numpy(x).to(tdt)
    got = ops._weight_int8pack_mm(xt.to("cuda:0"), torch.from_numpy(w).to("cuda:0"), torch.from_numpy(s).to("cuda:0"))
    y64 = (xt.double().numpy() @ w.astype(np.float64).T) * s.astype(np.float64)
    assert got.dtype == tdt and got.shape == (M, N)
    assert rel_err(got.float().cpu().numpy(), y64) < {"f32": 1e-4, "f16": 2e-3, "bf16": 1.6e-2}[dtype]
