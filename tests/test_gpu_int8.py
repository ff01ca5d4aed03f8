"""GPU parity: _int_mm (exact int32), _int8_mm_rescale and the fused dequant GEMM."""
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


def _rand_i8(rng, shape, lo=-128, hi=128):
    return rng.integers(lo, hi, size=shape).astype(np.int8)


# (M, K, N): generic path (odd sizes), small-M path, matrix-core path with ragged edges
SHAPES = [(5, 7, 3), (1, 1, 1), (64, 12, 32), (16, 1024, 1024), (64, 128, 32), (33, 257, 65),
          (129, 64, 65), (256, 4096, 128), (300, 208, 200), (128, 2560, 6912 // 8), (513, 80, 257),
          # decode kernel: 1..64 rows in slabs of 32 / 16, K a multiple of 128, ragged N, both widths of workgroup
          (1, 128, 40), (17, 256, 24), (48, 384, 72), (33, 4096, 100), (7, 11008, 64),
          (64, 256, 6150), (49, 128, 8200), (8, 384, 16400), (31, 256, 6144), (16, 128, 9000), (64, 512, 17),
          # 128-row tiles of the staggered kernel (65 rows and more where one round of them covers the problem)
          (130, 1024, 200), (300, 2048, 136), (65, 1152, 64), (257, 1280, 100), (33, 1024, 10248),
          # tiled kernel with the k range in slices (few tiles, long K), ragged last slice
          (130, 4096, 200), (300, 8192, 136), (65, 4608, 64), (257, 5120, 100), (300, 4224, 136),
          # one or two rows on the row kernel: a last chunk past K, several passes per channel, ragged N, the long rows
          # that fall back to the matrix-core kernel (more than 32768 k), and 3 / 4 rows (that kernel by default)
          (2, 4224, 10), (1, 20480, 13), (2, 32768, 9), (1, 36864, 8), (2, 4096, 8200), (1, 8192, 16390), (3, 4096, 50), (4, 256, 7),
          # all-in-flight decode kernel (3..32 rows, K = 2048..8192): 8 / 16 / 32 rows through LDS, every width of
          # workgroup, a dead last step (K = 2048, 5120), ragged N
          (3, 2048, 72), (8, 4096, 4104), (16, 4096, 264), (12, 5120, 136), (24, 4096, 520), (32, 2048, 40), (9, 8192, 72),
          (5, 4096, 16392)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("layout", ["weight_view", "contiguous"])
def test_int_mm_exact(ops, shape, layout):
    M, K, N = shape
    rng = np.random.default_rng(M * 31 + K * 7 + N)
    a = _rand_i8(rng, (M, K))
    w = _rand_i8(rng, (N, K))
    want = a.astype(np.int32) @ w.astype(np.int32).T
    np.testing.assert_array_equal(oracle.int_mm(a, w.T), want)
    wd = dev(w)
    b = wd.t() if layout == "weight_view" else wd.t().contiguous()
    got = ops._int_mm(dev(a), b)
    assert got.dtype == torch.int32 and got.shape == (M, N)
    np.testing.assert_array_equal(host(got), want)


def test_int_mm_unsigned_lhs_out_and_empty(ops):
    rng = np.random.default_rng(1)
    a = rng.integers(0, 256, size=(40, 100)).astype(np.uint8)
    b = _rand_i8(rng, (100, 24))
    want = a.astype(np.int32) @ b.astype(np.int32)
    np.testing.assert_array_equal(host(ops._int_mm(dev(a), dev(b))), want)
    out = torch.zeros(40, 24, dtype=torch.int32, device=DEV)
    assert ops._int_mm(dev(a), dev(b), out=out) is out
    np.testing.assert_array_equal(host(out), want)
    z = ops._int_mm(torch.empty(3, 0, dtype=torch.int8, device=DEV), torch.empty(0, 4, dtype=torch.int8, device=DEV))
    assert z.shape == (3, 4) and not z.any()
    assert ops._int_mm(torch.empty(0, 5, dtype=torch.int8, device=DEV), torch.empty(5, 4, dtype=torch.int8, device=DEV)).shape == (0, 4)
    with pytest.raises(Exception):
        ops._int_mm(torch.zeros(2, 2, device=DEV), torch.zeros(2, 2, dtype=torch.int8, device=DEV))
    with pytest.raises(Exception):
        ops._int_mm(torch.zeros(2, 3, dtype=torch.int8, device=DEV), torch.zeros(2, 2, dtype=torch.int8, device=DEV))


@pytest.mark.parametrize("shape", [(32, 4096, 11008), (128, 4096, 4096), (48, 11008, 4096), (512, 4096, 4096), (128, 8192, 8192)])
def test_int_mm_decode_and_sliced_kernels_at_model_sizes(ops, shape):
    """The decode kernel (32 rows per pass, both widths of workgroup), the 128-row tiles and the sliced tiled kernel
    (128 rows of 8192 x 8192) at real layer sizes, with the extremes in: exact against numpy, and against the single
    launch through the C ABI."""
    M, K, N = shape
    rng = np.random.default_rng(M + K + N)
    a = _rand_i8(rng, (M, K))
    w = _rand_i8(rng, (N, K))
    a[0, :] = -128
    w[N - 1, :] = -128
    a[M - 1, ::2] = 127
    want = a.astype(np.int32) @ w.astype(np.int32).T
    ad, wd = dev(a), dev(w)
    got = ops._int_mm(ad, wd.t())
    np.testing.assert_array_equal(host(got), want)
    from tensorplay_amd import _lib
    plain = torch.empty((M, N), dtype=torch.int32, device=DEV)
    rc = _lib.load().tpq_int_mm(ad.data_ptr(), 0, wd.data_ptr(), 1, K, plain.data_ptr(), M, K, N,
                                torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert torch.equal(plain, got)


def test_int_mm_extreme_values(ops):
    K = 6912
    a = np.full((130, K), -128, np.int8)
    w = np.full((70, K), -128, np.int8)
    got = host(ops._int_mm(dev(a), dev(w).t()))
    assert (got == 128 * 128 * K).all()


def test_rescale_bit_exact(ops):
    rng = np.random.default_rng(9)
    for M, N in [(37, 53), (16, 1024), (5, 7), (64, 4096)]:
        acc = rng.integers(-2**22, 2**22, size=(M, N)).astype(np.int32)
        rs = rng.uniform(1e-3, 1e-1, M).astype(np.float32)
        cs = rng.uniform(1e-4, 1e-2, N).astype(np.float32)
        got = ops._int8_mm_rescale(dev(acc), dev(rs).unsqueeze(-1), dev(cs).unsqueeze(-1))
        assert got.dtype == torch.float32
        np.testing.assert_array_equal(host(got), oracle.int8_mm_rescale(acc, rs, cs))
    with pytest.raises(ValueError):
        ops._int8_mm_rescale(torch.zeros(2, 2, device=DEV), torch.ones(2, device=DEV), torch.ones(2, device=DEV))


@pytest.mark.parametrize("out_dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("shape", [(16, 1024, 1024), (300, 208, 200), (5, 7, 3), (256, 512, 384), (40, 256, 36), (1, 4096, 64), (50, 256, 6160), (9, 128, 16390),
                                   (130, 1024, 200), (300, 2048, 136), (65, 1152, 66), (257, 1280, 100),
                                   # the ring kernel with one, two and three stages in all (which stage buffers are free for the
                                   # wavefronts' own epilogue depends on the count)
                                   (200, 128, 136), (300, 256, 264), (129, 384, 72),
                                   # all-in-flight decode kernel: runs of four channels stored with the scales fetched first
                                   (8, 4096, 264), (16, 2048, 4104), (27, 4096, 134), (5, 6144, 70)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_fused_dequant_bit_exact(ops, out_dtype, shape, with_bias):
    from gpu_util import TORCH_DT

    M, K, N = shape
    rng = np.random.default_rng(M + K + N)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    w = rng.normal(0, 0.02, (N, K)).astype(np.float32)
    bias = rng.normal(0, 0.01, N).astype(np.float32) if with_bias else None
    xq, xs = oracle.quantize_int8_rowwise(x)
    wq, ws = oracle.quantize_int8_rowwise(w)
    acc = oracle.int_mm(xq, wq.T)
    want = oracle.int8_mm_rescale(acc, xs, ws, bias=bias, out_dtype=out_dtype)
    got = ops.int8_mm_dequant(dev(xq), dev(wq), dev(xs), dev(ws), None if bias is None else dev(bias), TORCH_DT[out_dtype])
    np.testing.assert_array_equal(host(got), want)


@pytest.mark.parametrize("M", [1, 2, 3, 4])
@pytest.mark.parametrize("K,N", [(4224, 50), (12288, 7), (256, 4100)])
def test_row_kernel_one_to_four_rows(ops, M, K, N, kernel_override):
    """The kernel that streams the weight rows, for 1..4 activation rows (3 and 4 are not its default): raw sums exact,
    fused dequant equal to the oracle bit for bit in float32 and bfloat16, with a bias."""
    kernel_override("int8_row", 1)
    rng = np.random.default_rng(M * 5 + K + N)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    w = rng.normal(0, 0.02, (N, K)).astype(np.float32)
    bias = rng.normal(0, 0.01, N).astype(np.float32)
    xq, xs = oracle.quantize_int8_rowwise(x)
    wq, ws = oracle.quantize_int8_rowwise(w)
    acc = xq.astype(np.int32) @ wq.astype(np.int32).T
    np.testing.assert_array_equal(host(ops._int_mm(dev(xq), dev(wq).t())), acc)
    for out_dtype, tdt in (("f32", torch.float32), ("bf16", torch.bfloat16)):
        want = oracle.int8_mm_rescale(acc, xs, ws, bias=bias, out_dtype=out_dtype)
        got = ops.int8_mm_dequant(dev(xq), dev(wq), dev(xs), dev(ws), dev(bias), tdt)
        np.testing.assert_array_equal(host(got), want)


def test_dynamic_int8_linear_config1_end_to_end(ops):
    """CPU-plumbing configuration: M=16, K=1024, N=1024 fp32 with bias, quantize -> mm -> rescale."""
    rng = np.random.default_rng(2026)
    x = rng.normal(0, 1, (16, 1024)).astype(np.float32)
    w = rng.normal(0, 0.02, (1024, 1024)).astype(np.float32)
    b = rng.normal(0, 0.01, 1024).astype(np.float32)
    xq, xs = oracle.quantize_int8_rowwise(x)
    wq, ws = oracle.quantize_int8_rowwise(w)
    want = oracle.int8_mm_rescale(oracle.int_mm(xq, wq.T), xs, ws) + b
    a_q, a_s = ops._quantize_int8_rowwise(dev(x), 1e-5)
    w_q, w_s = ops._quantize_int8_rowwise(dev(w), 1e-5)
    out = ops._int8_mm_rescale(ops._int_mm(a_q, w_q.t()), a_s, w_s) + dev(b)
    np.testing.assert_array_equal(host(out), want)


def test_prefill_config3_full_size(ops):
    """M=2048, K=4096, N=4096 bf16 activations with outlier columns: int32 accumulators exact
    against an fp64 product on the device (exact for |acc| < 2^53) and against the oracle on a
    sample of rows; bf16 output equal to the oracle's rounding of the same accumulators."""
    M, K, N = 2048, 4096, 4096
    rng = np.random.default_rng(3)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    x[:, rng.choice(K, 41, replace=False)] *= 20.0
    w = rng.normal(0, 0.02, (N, K)).astype(np.float32)
    xb = cast_bits(x, "bf16")
    wb = cast_bits(w, "bf16")   # the reference casts the weight to the activation dtype first
    a_q, a_s = ops._quantize_int8_rowwise(dev(xb, "bf16"), 1e-5)
    w_q, w_s = ops._quantize_int8_rowwise(dev(wb, "bf16"), 1e-5)
    acc = ops._int_mm(a_q, w_q.t())
    ref = (a_q.double() @ w_q.double().t())
    assert torch.equal(acc.double(), ref)
    rows = np.arange(0, M, 171)
    aq_h, wq_h = host(a_q), host(w_q)
    np.testing.assert_array_equal(host(acc)[rows], oracle.int_mm_nk(aq_h[rows], wq_h))
    fused = ops.int8_mm_dequant(a_q, w_q, a_s, w_s, None, torch.bfloat16)
    want = oracle.int8_mm_rescale(host(acc)[rows], host(a_s)[rows], host(w_s), out_dtype="bf16")
    np.testing.assert_array_equal(host(fused)[rows], want)
    two_step = ops._int8_mm_rescale(acc, a_s, w_s).to(torch.bfloat16)
    assert torch.equal(fused, two_step)



# ---- the prepacked quantized linear in its general form (A12) ------------------------------------------------------

@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("shape", [(5, 7, 23), (5, 7, 64), (1, 8, 32), (33, 136, 4096), (300, 264, 2048), (2, 4104, 515), (64, 40, 65536)])
def test_packed_linear_general_form_bit_exact(ops, shape, unsigned, relu):
    """acc = x.w - xz off[n] - wz[n] sum(x) + K xz wz[n] in integers, fmaf(float(acc), float(xs) * ws[n], bias[n]):
    bit-exact with the oracle's restatement of QuantPacked.cpp:420-516 (linear, float output), signed and unsigned
    activation codes, rows that are and are not multiples of 32 long, the matrix-core and the generic product."""
    M, N, K = shape
    rng = np.random.default_rng(M * 31 + N + K + unsigned)
    x = rng.integers(0 if unsigned else -128, 256 if unsigned else 128, size=(M, K)).astype(np.uint8 if unsigned else np.int8)
    w = rng.integers(-128, 128, size=(N, K)).astype(np.int8)
    xs, xz = 0.021, (137 if unsigned else -13)
    scales = rng.uniform(0.004, 0.04, N).astype(np.float32)
    zps = rng.integers(-5, 6, N).astype(np.int64)
    bias = rng.normal(0, 0.7, N).astype(np.float32)
    packed_ref, offsets_ref = oracle.weight_prepack(w)
    packed, offsets = ops._quantized_weight_prepack(torch.from_numpy(w).to(DEV))
    np.testing.assert_array_equal(packed.cpu().numpy(), packed_ref)
    np.testing.assert_array_equal(offsets.cpu().numpy(), offsets_ref)
    for b in (bias, None):
        want = oracle.packed_run_linear_float(x, xs, xz, packed_ref, offsets_ref, scales, zps, b, K)
        if relu:
            want = np.maximum(want, 0.0)
        got = ops._quantized_packed_run_linear(torch.from_numpy(x).to(DEV), xs, xz, packed, offsets, torch.from_numpy(scales).to(DEV),
                                               torch.from_numpy(zps).to(DEV), None if b is None else torch.from_numpy(b).to(DEV), K, relu=relu)
        np.testing.assert_array_equal(got.cpu().numpy(), want)
    # the hot path's special case: unit scales, zero zero-points, no bias = float(_int_mm)
    plain = ops._quantized_packed_run_linear(torch.from_numpy(x).to(DEV), 1.0, 0, packed, offsets, torch.ones(N, device=DEV),
                                             torch.zeros(N, dtype=torch.int64, device=DEV), None, K)
    np.testing.assert_array_equal(plain.cpu().numpy(), (x.astype(np.int64) @ w.astype(np.int64).T).astype(np.float32))
