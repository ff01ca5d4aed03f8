"""GPU parity: int4 device pack (bit-exact) and the int4 weight-only matmul (tolerance).

Tolerances (stated by the target of this build): outputs in fp16/bf16 within 1e-2 of the
reference formulation; against an fp64 evaluation of the same quantized weights the fp16
output stays within 1e-3 (normwise), bf16 within 1e-2 (its own rounding is 2^-8).
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import DEV, TORCH_DT, assert_close_norm, cast_bits, dev, from_bits, host, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from tensorplay_amd import ops as _ops

    return _ops


def asym_quant(w, group):
    """Asymmetric uint4 group quantizer of the benchmark configuration:
    s = (max-min)/15, q = clamp(round((w-min)/s), 0, 15), zero = min + 8 s."""
    N, K = w.shape
    wg = w.reshape(N, K // group, group)
    lo, hi = wg.min(-1), wg.max(-1)
    s = np.maximum((hi - lo) / 15.0, 1e-8).astype(np.float32)
    q = np.clip(np.rint((wg - lo[..., None]) / s[..., None]), 0, 15).astype(np.int32).reshape(N, K)
    z = (lo + 8 * s).astype(np.float32)
    return q, np.ascontiguousarray(np.stack([s.T, z.T], axis=-1))  # [K/g, N, 2]


@pytest.mark.parametrize("inner", [2, 4, 8])
@pytest.mark.parametrize("shape", [(16, 64), (8, 32), (24, 160), (13, 70), (40, 256), (64, 4096), (1000, 130)])
def test_pack_bit_exact(ops, inner, shape):
    rng = np.random.default_rng(shape[0] * 1000 + shape[1] + inner)
    codes = rng.integers(0, 16, size=shape, dtype="int32")
    got = ops._convert_weight_to_int4pack(dev(codes), inner)
    want = oracle.int4_pack_tc(codes, inner)
    assert got.dtype == torch.int32 and tuple(got.shape) == want.shape
    np.testing.assert_array_equal(host(got), want)


def test_pack_full_size_round_trip(ops):
    N, K = 11008, 4096
    rng = np.random.default_rng(0)
    codes = rng.integers(0, 16, size=(N, K), dtype="int32")
    packed = host(ops._convert_weight_to_int4pack(dev(codes), 2))
    assert packed.shape == (1376, 128, 32, 1)
    np.testing.assert_array_equal(oracle.int4_unpack_tc(packed, K), codes)


def test_pack_errors(ops):
    with pytest.raises(ValueError):
        ops._convert_weight_to_int4pack(torch.zeros(8, 33, dtype=torch.int32, device=DEV), 2)
    with pytest.raises(ValueError):
        ops._convert_weight_to_int4pack(torch.zeros(8, 32, dtype=torch.int32, device=DEV), 3)
    with pytest.raises(ValueError):
        ops._convert_weight_to_int4pack(torch.zeros(8, dtype=torch.int32, device=DEV), 2)
    assert ops._convert_weight_to_int4pack(torch.zeros(0, 32, dtype=torch.int32, device=DEV), 2).shape == (0, 1, 32, 1)


CASES = [  # M, N, K, group
    (1, 64, 256, 128), (1, 72, 128, 128), (4, 40, 128, 32), (16, 128, 512, 64), (3, 200, 384, 128),
    (2, 64, 4096, 128), (5, 24, 96, 32), (1, 16, 70, 32), (7, 136, 1024, 64),
    # matrix-core decode kernel: 5..16 rows (64-channel workgroups, partial last one), slabs of 16 plus a last row
    (16, 72, 256, 128), (9, 136, 1024, 128), (17, 64, 256, 128), (33, 40, 384, 128), (8, 200, 2048, 128),
    # slabs of 32 rows (two row blocks per workgroup), partial last block, every width of workgroup
    (24, 136, 512, 128), (64, 72, 1024, 128), (50, 200, 256, 128), (130, 64, 384, 128), (81, 40, 1152, 128),
    (32, 6152, 256, 128), (31, 10248, 128, 128), (19, 5128, 256, 128), (128, 8200, 128, 128),
    # groups of 32 / 64: dequantized in registers (fp16, bf16), every shape of workgroup (by N and rows), one row too
    (4, 8200, 256, 32), (12, 8192, 384, 64), (2, 48, 640, 32), (16, 24, 128, 64),
    (9, 6152, 256, 32), (16, 10248, 128, 64), (1, 4104, 256, 32), (3, 10240, 256, 32), (1, 10240, 128, 64),
    # one row on the column-per-lane kernel with its branch-free body: one, two and three chunks per wavefront
    # (K = 2048, 4096, 6144), every group size, a partial last column block
    (1, 10248, 2048, 128), (1, 10264, 4096, 32), (1, 10240, 4096, 64), (1, 10300 // 8 * 8, 6144, 128),
]


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("M,N,K,group", CASES)
def test_mm_matches_oracle(ops, dtype, M, N, K, group):
    rng = np.random.default_rng(M * 100003 + N * 101 + K + group)
    Kg = (K + group - 1) // group * group
    w = rng.normal(0, 0.02, (N, Kg)).astype(np.float32)
    codes, sz = asym_quant(w, group)
    codes = codes[:, :K]
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    xb, szb = cast_bits(x, dtype), cast_bits(sz, dtype)
    packed = oracle.int4_pack_tc(codes, 2)
    got = ops._weight_int4pack_mm(dev(xb, dtype), dev(packed), group, dev(szb, dtype))
    assert got.dtype == TORCH_DT[dtype] and got.shape == (M, packed.shape[0] * 8)
    got32 = got.float().cpu().numpy()
    ref_dev = oracle.to_f32(oracle.int4_mm_tc(xb, dtype, packed, szb, group, round_w=True), dtype)
    _, y64 = oracle.int4_mm_tc(xb, dtype, packed, szb, group, round_w=False, want_f64=True)
    # the stated tolerance, 1e-2 normwise and elementwise, against the reference's CPU kernel
    assert_close_to_cpu_formulation(got32, xb, dtype, codes, szb, group)
    # secondary: the reference's device formulation, which rounds every weight to the activation dtype twice; for bf16
    # (2^-8 per rounding) two correct evaluations of it differ by more than 1e-2 on a few of ~10^5 outputs, so the widest
    # bf16 cases (and long sums, K >= 4096) get 1.5e-2 in this check only
    assert_close_norm(got32, ref_dev, 1.5e-2 if dtype == "bf16" and (M * N > 50000 or K >= 4096) else 1e-2, "vs the device formulation (secondary)")
    # fp32-accumulate comparison against the exact sums
    tol = {"f16": 1e-3, "bf16": 1e-2, "f32": 1e-5}[dtype]
    assert rel_err(got32, y64) < tol


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,N,K,group", [(113, 136, 512, 128), (128, 72, 128, 128), (200, 8200, 256, 64), (257, 264, 384, 32),
                                         (300, 520, 1024, 128), (640, 8, 256, 128), (129, 4096, 4096, 128)])
def test_mm_tiled_kernel_matches_oracle(ops, dtype, M, N, K, group):
    """113 rows and more through the C ABI: the tiled kernel (both shapes of workgroup, ragged M and N, every group size),
    against the oracle to the bounds of test_mm_matches_oracle, and against the decode kernels' rows."""
    from tensorplay_amd import _lib
    rng = np.random.default_rng(M * 7 + N * 3 + K + group)
    codes, sz = asym_quant(rng.normal(0, 0.02, (N, K)).astype(np.float32), group)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    xb, szb = cast_bits(x, dtype), cast_bits(sz, dtype)
    packed = oracle.int4_pack_tc(codes, 2)
    xd, pd, sd = dev(xb, dtype), dev(packed), dev(szb, dtype)
    out = torch.empty((M, N), dtype=TORCH_DT[dtype], device=DEV)
    tag = {"f16": _lib.F16, "bf16": _lib.BF16}[dtype]
    rc = _lib.load().tpq_int4_mm(xd.data_ptr(), tag, M, K, pd.data_ptr(), 2, N, group, sd.data_ptr(), out.data_ptr(),
                                 torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.last_error()
    got32 = out.float().cpu().numpy()
    ref_dev = oracle.to_f32(oracle.int4_mm_tc(xb, dtype, packed, szb, group, round_w=True), dtype)
    _, y64 = oracle.int4_mm_tc(xb, dtype, packed, szb, group, round_w=False, want_f64=True)
    assert_close_to_cpu_formulation(got32, xb, dtype, codes, szb, group)
    # secondary (device formulation, two roundings per weight: the widest bf16 cases get 1.5e-2 in this check only)
    assert_close_norm(got32, ref_dev, 1.5e-2 if dtype == "bf16" and (M * N > 50000 or K >= 4096) else 1e-2, "vs the device formulation (secondary)")
    assert rel_err(got32, y64) < {"f16": 1e-3, "bf16": 1e-2}[dtype]
    few = ops._weight_int4pack_mm(xd[:16], pd, group, sd).float().cpu().numpy()   # the decode kernel on the first rows
    # two kernels, each within its bound of the oracle (bf16: the decode kernel rounds small-group weights once, this one twice)
    assert_close_norm(got32[:16], few, 2e-2 if dtype == "bf16" else 1e-2, "vs the decode kernel (cross-check of two kernels, each within 1e-2 of the CPU formulation)")


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,N,K,group", [(40, 264, 2048, 128), (128, 520, 4096, 128), (200, 72, 11008, 128), (113, 264, 1024, 64),
                                         (64, 2048, 2048, 128), (255, 136, 3072, 32), (96, 4096, 11008, 128)])
def test_mm_tiled_kernel_with_slices_of_k(ops, dtype, M, N, K, group):
    """33 .. 256 rows with a workspace: where the tiled kernel would leave most compute units idle the steps of K go to
    several slices, whose fp32 sums meet in the workspace in slice order.  Against the CPU formulation and the exact
    sums to the bounds of test_mm_matches_oracle, twice in a row into the same workspace bit for bit, and against the
    same call without workspace (one slice or the 32-row slabs: other order of the sums only)."""
    from tensorplay_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(M * 5 + N * 3 + K + group)
    codes, sz = asym_quant(rng.normal(0, 0.02, (N, K)).astype(np.float32), group)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    xb, szb = cast_bits(x, dtype), cast_bits(sz, dtype)
    packed = oracle.int4_pack_tc(codes, 2)
    xd, pd, sd = dev(xb, dtype), dev(packed), dev(szb, dtype)
    tag = {"f16": _lib.F16, "bf16": _lib.BF16}[dtype]
    need = lib.tpq_int4_mm_rows_workspace_bytes(M, N, K)
    assert need >= lib.tpq_int4_mm_workspace_bytes(N)
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for _ in range(2):
        out = torch.full((M, N), float("nan"), dtype=TORCH_DT[dtype], device=DEV)
        rc = lib.tpq_int4_mm_ws(xd.data_ptr(), tag, M, K, pd.data_ptr(), 2, N, group, sd.data_ptr(), out.data_ptr(), ws.data_ptr(), need, stream)
        assert rc == 0, _lib.last_error()
        outs.append(out)
    assert torch.equal(outs[0], outs[1])
    got32 = outs[0].float().cpu().numpy()
    _, y64 = oracle.int4_mm_tc(xb, dtype, packed, szb, group, round_w=False, want_f64=True)
    assert_close_to_cpu_formulation(got32, xb, dtype, codes, szb, group)
    assert rel_err(got32, y64) < {"f16": 1e-3, "bf16": 1e-2}[dtype]
    plain = torch.empty((M, N), dtype=TORCH_DT[dtype], device=DEV)
    rc = lib.tpq_int4_mm(xd.data_ptr(), tag, M, K, pd.data_ptr(), 2, N, group, sd.data_ptr(), plain.data_ptr(), stream)
    assert rc == 0, _lib.last_error()
    assert_close_norm(got32, plain.float().cpu().numpy(), 2e-2 if dtype == "bf16" else 1e-2, "vs the call without workspace")
    # the counters at the front of the workspace are zero again: a decode call may share it
    assert int(ws[:16384].view(torch.int32).abs().sum()) == 0


@pytest.mark.parametrize("M", [1, 4, 16])
def test_mm_config2_full_size(ops, M):
    """M x 4096 x 11008, group 128, fp16: the decode configuration at its real size."""
    N, K, g = 11008, 4096, 128
    rng = np.random.default_rng(42)
    w = rng.normal(0, 0.02, (N, K)).astype(np.float32)
    codes, sz = asym_quant(w, g)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    xb, szb = cast_bits(x, "f16"), cast_bits(sz, "f16")
    packed_d = ops._convert_weight_to_int4pack(dev(codes), 2)
    packed = host(packed_d)
    np.testing.assert_array_equal(packed, oracle.int4_pack_tc(codes, 2))
    got = ops._weight_int4pack_mm(dev(xb, "f16"), packed_d, g, dev(szb, "f16")).float().cpu().numpy()
    ref, y64 = oracle.int4_mm_tc(xb, "f16", packed, szb, g, round_w=False, want_f64=True)
    assert rel_err(got, y64) < 1e-3
    assert_close_norm(got, oracle.to_f32(oracle.int4_mm_tc(xb, "f16", packed, szb, g, round_w=True), "f16"), 1e-2)
    # linearity in x: doubling the activations doubles the result exactly (power of two)
    got2 = ops._weight_int4pack_mm(dev(cast_bits(2 * from_bits(xb, "f16").float().numpy(), "f16"), "f16"), packed_d, g, dev(szb, "f16"))
    got2 = got2.float().cpu().numpy()
    normal = np.abs(got) > 1e-3  # doubling is exact only above fp16's subnormal range
    np.testing.assert_array_equal(got2[normal], 2 * got[normal])


def test_mm_errors(ops):
    x = torch.zeros(2, 64, dtype=torch.float16, device=DEV)
    packed = torch.zeros(2, 2, 32, 1, dtype=torch.int32, device=DEV)
    sz = torch.zeros(2, 16, 2, dtype=torch.float16, device=DEV)
    with pytest.raises(TypeError):
        ops._weight_int4pack_mm(x, packed.to(torch.uint8), 32, sz)
    with pytest.raises(ValueError):
        ops._weight_int4pack_mm(x, packed, 16, sz)
    with pytest.raises(ValueError):
        ops._weight_int4pack_mm(x, packed, 32, sz[:1])
    with pytest.raises(ValueError):
        ops._weight_int4pack_mm(x[:, :32], packed, 32, sz)
    assert ops._weight_int4pack_mm(x[:0], packed, 32, sz).shape == (0, 16)


@pytest.mark.parametrize("columns,half_split", [(64, True), (32, True), (32, False)])
@pytest.mark.parametrize("shape", [(16, 64), (80, 128), (128, 256), (48, 70), (256, 4096)])
def test_cpu_layout_pack_and_conversion(ops, columns, half_split, shape):
    """The CPU layout written on the GPU equals the oracle's (itself byte-equal to PyTorch's CPU pack), and
    converting it to the device layout gives what the device pack writes from the codes."""
    N, K = shape
    rng = np.random.default_rng(N * 31 + K)
    codes = rng.integers(0, 16, size=(N, K), dtype=np.int32)
    cpu_layout = ops._convert_weight_to_int4pack_for_cpu(dev(codes), 2, block_cols=columns, half_split=half_split)
    np.testing.assert_array_equal(host(cpu_layout), oracle.int4_pack_cpu(codes, columns, half_split))
    converted = ops.int4pack_cpu_to_device(cpu_layout, block_cols=columns, half_split=half_split)
    np.testing.assert_array_equal(host(converted), oracle.int4_pack_tc(codes, 2))


def test_cpu_layout_equals_torch_cpu_pack(ops):
    rng = np.random.default_rng(124)
    codes = rng.integers(0, 16, size=(64, 256), dtype="int32")
    want = torch._convert_weight_to_int4pack_for_cpu(torch.tensor(codes), 2).numpy()
    np.testing.assert_array_equal(host(ops._convert_weight_to_int4pack_for_cpu(dev(codes), 2)), want)
    with pytest.raises(ValueError):
        ops._convert_weight_to_int4pack_for_cpu(torch.zeros(8, 32, dtype=torch.int32, device=DEV), 2)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("N,K,group", [(64, 256, 128), (40, 96, 32), (136, 1024, 64), (8, 70, 32), (264, 4096, 128), (16, 2080, 32)])
def test_dequantize_bit_exact(ops, dtype, N, K, group):
    """Dense weight from the packed layout: the reference's dequantize kernel, bit for bit."""
    rng = np.random.default_rng(N + K + group)
    Kg = (K + group - 1) // group * group
    codes, sz = asym_quant(rng.normal(0, 0.02, (N, Kg)).astype(np.float32), group)
    codes = codes[:, :K]
    szb = cast_bits(sz, dtype)
    packed = oracle.int4_pack_tc(codes, 2)
    got = ops._int4_dequantize(dev(packed), 2, packed.shape[0] * 8, K, group, dev(szb, dtype))
    want = oracle.int4_dequantize_tc(packed, szb, dtype, K, group)
    np.testing.assert_array_equal(host(got), want)


def test_dequantize_bf16_non_finite_scale(ops):
    """An infinite scale gives +-inf and, for code 8, NaN: the dense bf16 weight carries the same bit patterns as the
    scalar conversion of the oracle (NaN = 0x7FC0)."""
    rng = np.random.default_rng(77)
    N, K, group = 16, 256, 128
    codes, sz = asym_quant(rng.normal(0, 0.02, (N, K)).astype(np.float32), group)
    codes[3, :16] = np.arange(16)
    sz[0, 3, 0] = np.inf
    sz[1, 5, 1] = np.nan
    szb = cast_bits(sz, "bf16")
    packed = oracle.int4_pack_tc(codes, 2)
    got = ops._int4_dequantize(dev(packed), 2, N, K, group, dev(szb, "bf16"))
    want = oracle.int4_dequantize_tc(packed, szb, "bf16", K, group)
    np.testing.assert_array_equal(host(got), want)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
def test_mm_many_rows_takes_the_dense_route(ops, dtype):
    """More than INT4_PREFILL_ROWS rows: dequantise + one dense GEMM (tpq_dense_mm where K allows), the reference's device formulation."""
    M, N, K, group = ops.INT4_PREFILL_ROWS + 37, 136, 512, 128
    rng = np.random.default_rng(77)
    codes, sz = asym_quant(rng.normal(0, 0.02, (N, K)).astype(np.float32), group)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    xb, szb = cast_bits(x, dtype), cast_bits(sz, dtype)
    packed = oracle.int4_pack_tc(codes, 2)
    got = ops._weight_int4pack_mm(dev(xb, dtype), dev(packed), group, dev(szb, dtype)).float().cpu().numpy()
    ref_dev = oracle.to_f32(oracle.int4_mm_tc(xb, dtype, packed, szb, group, round_w=True), dtype)
    assert_close_norm(got, ref_dev, 1e-2, "vs reference formulation")
    _, y64 = oracle.int4_mm_tc(xb, dtype, packed, szb, group, round_w=False, want_f64=True)
    assert rel_err(got, y64) < {"f16": 2e-3, "bf16": 1e-2, "f32": 1e-4}[dtype]


def test_mm_float32_many_rows_on_the_library_gemm(ops):
    """float32 activations from DENSE_F32_ROWS rows on: dequantise, then the library's tile kernel with float32 MFMAs
    (no framework GEMM); against the reference's formulation and the exact sums."""
    M, N, K, group = ops.DENSE_F32_ROWS + 5, 264, 1024, 128
    rng = np.random.default_rng(78)
    codes, sz = asym_quant(rng.normal(0, 0.02, (N, K)).astype(np.float32), group)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    xb, szb = cast_bits(x, "f32"), cast_bits(sz, "f32")
    packed = oracle.int4_pack_tc(codes, 2)
    calls = []
    real = torch.matmul
    torch.matmul = lambda *a, **k: calls.append(1) or real(*a, **k)
    try:
        got = ops._weight_int4pack_mm(dev(xb, "f32"), dev(packed), group, dev(szb, "f32")).float().cpu().numpy()
    finally:
        torch.matmul = real
    assert not calls, "the many-row float32 route went through torch.matmul"
    ref_dev = oracle.to_f32(oracle.int4_mm_tc(xb, "f32", packed, szb, group, round_w=True), "f32")
    assert_close_norm(got, ref_dev, 1e-4, "vs reference formulation")
    _, y64 = oracle.int4_mm_tc(xb, "f32", packed, szb, group, round_w=False, want_f64=True)
    assert rel_err(got, y64) < 1e-5


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_mm_prefill_block_matches_cpu_formulation(ops, dtype):
    """2048 rows of 4096 -> 11008, the prefill block of the model the decode numbers are quoted on: dequantise, then
    the library's dense tile kernel (no framework GEMM on this route)."""
    M, N, K, group = 2048, 11008, 4096, 128
    rng = np.random.default_rng(2048)
    codes, sz = asym_quant(rng.normal(0, 0.02, (N, K)).astype(np.float32), group)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    xb, szb = cast_bits(x, dtype), cast_bits(sz, dtype)
    packed = ops._convert_weight_to_int4pack(torch.from_numpy(codes).to(DEV), 2)
    calls = []
    real = torch.matmul
    torch.matmul = lambda *a, **k: calls.append(1) or real(*a, **k)
    try:
        got = ops._weight_int4pack_mm(dev(xb, dtype), packed, group, dev(szb, dtype)).float().cpu().numpy()
    finally:
        torch.matmul = real
    assert not calls, "the many-row route went through torch.matmul"
    assert_close_to_cpu_formulation(got, xb, dtype, codes, szb, group)


# ---- fusions around the decode matmul --------------------------------------------------------------

FLIGHT_CASES = [  # M, N, K, group: the all-in-flight matrix-core kernel (K >= 2048, 2..16 rows, groups of 128)
    (2, 72, 2048, 128),      # 16 steps: one per wavefront, the second one dead; half a block at the end
    (3, 200, 4096, 128),     # four rows through LDS
    (5, 4104, 4096, 128),    # eight rows, 257 blocks: two per workgroup
    (8, 11008, 4096, 128),   # the decode configuration: three blocks per workgroup
    (4, 16392, 4096, 128),   # more blocks than four per compute unit cover in one pass
    (9, 136, 4096, 128),     # 16 rows through LDS, one step resident at a time
    (16, 264, 5120, 128),    # 40 steps: three per wavefront, the third dead for half of them
    (4, 520, 6144, 128),     # 48 steps
    (7, 136, 8192, 128),     # four steps per wavefront
    (8, 4104, 11008, 128),   # 86 steps: six per wavefront, one block per workgroup
    (13, 72, 11008, 128),
    (6, 264, 14336, 128),    # seven steps per wavefront
    (12, 264, 14336, 128),   # (that many steps at more than eight rows: the loop kernel)
    # 17..32 rows: two blocks of 16 rows against the same weight registers (K = 3072..4096), every width of workgroup
    # that takes it, a partial second block, a partial last channel block, and a slab of 32 plus a rest
    (17, 72, 3072, 128), (32, 264, 4096, 128), (25, 136, 3584, 128), (31, 8200, 4096, 128), (20, 11008, 4096, 128),
    (50, 72, 4096, 128), (29, 136, 5120, 128), (32, 4096, 6144, 128),   # three steps per wavefront, one block per workgroup
]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,N,K,group", FLIGHT_CASES)
def test_mm_all_in_flight_kernel_matches_oracle(ops, dtype, M, N, K, group):
    rng = np.random.default_rng(M * 977 + N * 13 + K + group)
    codes, sz = asym_quant(rng.normal(0, 0.02, (N, K)).astype(np.float32), group)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    xb, szb = cast_bits(x, dtype), cast_bits(sz, dtype)
    packed = ops._convert_weight_to_int4pack(torch.from_numpy(codes).to(DEV), 2)
    got32 = ops._weight_int4pack_mm(dev(xb, dtype), packed, group, dev(szb, dtype)).float().cpu().numpy()
    assert got32.shape == (M, N)
    # the oracle on whole packed tiles of eight channels, first and last included
    tiles = _tile_subset(rng, N // 8, 40)
    cols = (tiles[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
    sub = oracle.int4_pack_tc(codes[cols], 2)
    ref_dev = oracle.to_f32(oracle.int4_mm_tc(xb, dtype, sub, szb[:, cols], group, round_w=True), dtype)
    _, y64 = oracle.int4_mm_tc(xb, dtype, sub, szb[:, cols], group, round_w=False, want_f64=True)
    assert_close_to_cpu_formulation(got32, xb, dtype, codes, szb, group)
    assert_close_norm(got32[:, cols], ref_dev, 1.5e-2 if dtype == "bf16" else 1e-2, "vs the device formulation (secondary)")
    assert rel_err(got32[:, cols], y64) < {"f16": 1e-3, "bf16": 1e-2}[dtype]
    # every channel: against the same kernel family at one row more or less is no check, so the rest of the columns
    # are held against a float64 product of the dequantized weights
    s64 = szb if dtype == "f32" else oracle.to_f32(szb, dtype)
    wq = (codes - 8) * np.repeat(s64[:, :, 0].T, group, axis=1).astype(np.float64) + np.repeat(s64[:, :, 1].T, group, axis=1)
    want = oracle.to_f32(xb, dtype).astype(np.float64) @ wq.T
    assert rel_err(got32, want) < {"f16": 1e-3, "bf16": 1e-2}[dtype]


def _fused_case(rng, M, N, K, tdt):
    codes = rng.integers(0, 16, (N, K)).astype(np.int32)
    sz = np.stack([rng.uniform(0.005, 0.02, (K // 128, N)), rng.uniform(-0.05, 0.05, (K // 128, N))], axis=-1).astype(np.float32)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(tdt)
    return codes, torch.from_numpy(sz).to(tdt), x


def _tile_subset(rng, n_tiles, count):
    """Indices of up to `count` packed tiles (8 channels each), sorted, always with the first and the last."""
    if n_tiles <= count:
        return np.arange(n_tiles)
    inner = rng.choice(np.arange(1, n_tiles - 1), size=count - 2, replace=False)
    return np.sort(np.concatenate([[0, n_tiles - 1], inner]))


def assert_close_to_cpu_formulation(got32, xb, dtype, codes, szb, group, what=""):
    """The comparison that carries the stated tolerance (max relative error 1e-2 for 16-bit outputs, normwise and
    elementwise): against the reference's CPU kernel, w = fma(code - 8, scale, zero) in float32, float32 fma over k in
    order, one cast (p10/src/backend/cpu/QuantizedElementwiseKernels.cpp:470-479; oracle.int4_mm_cpu restates it and is
    bit-exact with torch._weight_int4pack_mm_for_cpu).  On a subset of rows and of whole 16-channel blocks that keeps the
    scalar oracle within a second: first and last block and first and last row always included."""
    M, K = xb.shape
    N = codes.shape[0]
    rng = np.random.default_rng(N * 31 + K + M)
    rows = np.arange(M) if M <= 4 else np.unique(np.concatenate([[0, M - 1], rng.choice(M, 2, replace=False)]))
    budget = max(2, int(3e7 // (len(rows) * K * 16)))
    blocks = _tile_subset(rng, (N + 15) // 16, budget)
    cols = np.minimum((blocks[:, None] * 16 + np.arange(16)[None, :]).reshape(-1), N - 1)  # a ragged last block repeats the last channel
    packed_cpu = oracle.int4_pack_cpu(np.ascontiguousarray(codes[cols]))
    ref = oracle.to_f32(oracle.int4_mm_cpu(np.ascontiguousarray(xb[rows]), dtype, packed_cpu, np.ascontiguousarray(szb[:, cols]), group), dtype)
    assert_close_norm(got32[np.ix_(rows, cols)], ref, {"f16": 1e-2, "bf16": 1e-2, "f32": 1e-4}[dtype], what or "vs the reference's CPU formulation")


@pytest.mark.parametrize("tdt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 64, 256), (8, 136, 512), (16, 4096, 1024), (19, 48, 384),
                                   (8, 264, 4096), (3, 72, 11008), (12, 4104, 4096),  # the all-in-flight kernel
                                   (24, 136, 4096), (32, 4104, 3072)])               # ... with two blocks of 16 rows
def test_mm_add_equals_the_two_ops(ops, tdt, M, N, K):
    """out = residual + x.W^T with both roundings of the separate ops: equal bit for bit whenever the matmul
    runs on the same kernel (rows > 1), within one rounding of it otherwise."""
    rng = np.random.default_rng(M * 1000 + N)
    codes, sz, x = _fused_case(rng, M, N, K, tdt)
    packed = ops._convert_weight_to_int4pack(torch.from_numpy(codes).to(DEV), 2)
    res = torch.from_numpy(rng.standard_normal((M, N)).astype(np.float32)).to(tdt).to(DEV)
    got = ops.int4pack_mm_add(x.to(DEV), packed, 128, sz.to(DEV), res)
    want = res + ops._weight_int4pack_mm(x.to(DEV), packed, 128, sz.to(DEV))
    if M > 1 and M % 16 != 1:
        assert torch.equal(got, want)
    else:
        assert_close_norm(got.float().cpu().numpy(), want.float().cpu().numpy(), 4e-3 if tdt == torch.float16 else 2e-2)


@pytest.mark.parametrize("tdt,tol", [(torch.float16, 2e-3), (torch.bfloat16, 1.6e-2)])
@pytest.mark.parametrize("M,N,K", [(1, 64, 256), (8, 136, 512), (16, 1024, 1024), (19, 48, 384),
                                   # the all-in-flight kernel: 4 / 8 / 16 rows through LDS, every width of workgroup, a partial block
                                   (2, 72, 4096), (5, 136, 2048), (12, 200, 4096), (8, 4104, 4096), (7, 8200, 4096)])
def test_mm_swiglu_against_oracle(ops, tdt, tol, M, N, K):
    """silu_mul(T(x.Wg^T), T(x.Wu^T)): the oracle's two device-layout products rounded to T, then
    gate * sigmoid(gate) * up in float32 (p10/src/backend/cpu/PointwiseKernels.cpp:1466-1478)."""
    rng = np.random.default_rng(M * 77 + N)
    tag = "f16" if tdt == torch.float16 else "bf16"
    cg, szg, x = _fused_case(rng, M, N, K, tdt)
    cu, szu, _ = _fused_case(rng, M, N, K, tdt)
    pg = ops._convert_weight_to_int4pack(torch.from_numpy(cg).to(DEV), 2)
    pu = ops._convert_weight_to_int4pack(torch.from_numpy(cu).to(DEV), 2)
    got = ops.int4pack_mm_swiglu(x.to(DEV), pg, pu, 128, szg.to(DEV), szu.to(DEV))
    g = ops._weight_int4pack_mm(x.to(DEV), pg, 128, szg.to(DEV)).float()
    u = ops._weight_int4pack_mm(x.to(DEV), pu, 128, szu.to(DEV)).float()
    unfused = (g * torch.sigmoid(g) * u).to(tdt)
    assert_close_norm(got.float().cpu().numpy(), unfused.float().cpu().numpy(), tol)
    # and against the CPU oracle's products
    og = oracle.to_f32(oracle.int4_mm_tc(host(x), tag, oracle.int4_pack_tc(cg, 2), host(szg), 128), tag)
    ou = oracle.to_f32(oracle.int4_mm_tc(host(x), tag, oracle.int4_pack_tc(cu, 2), host(szu), 128), tag)
    want = og * (1.0 / (1.0 + np.exp(-og))) * ou
    assert_close_norm(got.float().cpu().numpy(), want, 2 * tol)


@pytest.mark.parametrize("tdt,tol", [(torch.float16, 1e-3), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("M,K,widths", [(1, 256, (64,)), (8, 512, (136, 136, 136)), (16, 1024, (1024, 256, 256)),
                                        (19, 384, (48, 8, 200, 16)), (8, 4096, (4096, 4096, 4096)), (4, 4096, (11008, 11008)),
                                        # the all-in-flight kernel: blocks of different weights in one workgroup
                                        (5, 4096, (72, 8, 200, 16)), (9, 11008, (136, 264)), (3, 8192, (4104, 24, 4096)),
                                        # ... 17..32 rows as two blocks of 16 in one launch, a slab of 32 plus a rest
                                        (32, 4096, (4096, 4096, 4096)), (21, 3072, (72, 8, 200, 16)), (45, 4096, (136, 264))])
def test_mm_multi_equals_separate_products(ops, tdt, tol, M, K, widths):
    """Several weights on one input in one launch: every output against the separate op (the same kernel; the order
    in which the wavefronts' partial sums are added may differ with the workgroup shape) and against the oracle."""
    rng = np.random.default_rng(M * 31 + K + len(widths))
    tag = "f16" if tdt == torch.float16 else "bf16"
    cases = [_fused_case(rng, M, n, K, tdt) for n in widths]
    x = cases[0][2].to(DEV)
    packed = [ops._convert_weight_to_int4pack(torch.from_numpy(c).to(DEV), 2) for c, _, _ in cases]
    szs = [sz.to(DEV) for _, sz, _ in cases]
    got = ops.int4pack_mm_multi(x, packed, 128, szs)
    assert len(got) == len(widths)
    for (codes, sz, _), p, szd, y, n in zip(cases, packed, szs, got, widths):
        assert tuple(y.shape) == (M, n) and y.dtype == tdt
        assert_close_norm(y.float().cpu().numpy(), ops._weight_int4pack_mm(x, p, 128, szd).float().cpu().numpy(), tol)
        # against the oracle on a subset of the output channels (whole packed tiles of 8, first and last included)
        tiles = _tile_subset(rng, n // 8, 32)
        cols = (tiles[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
        want = oracle.to_f32(oracle.int4_mm_tc(host(x), tag, oracle.int4_pack_tc(codes[cols], 2), host(sz)[:, cols], 128), tag)
        assert_close_norm(y.float().cpu().numpy()[:, cols], want, 2 * tol)


def _rms_norm_bits(x_bits, g_bits, tag, eps):
    """The reference's rms_norm in numpy float32 (tensorplay/nn/functional.py:2350-2372), rounded to the dtype."""
    x = oracle.to_f32(x_bits, tag)
    inv = (1.0 / np.sqrt((x * x).mean(-1, keepdims=True, dtype=np.float32) + np.float32(eps))).astype(np.float32)
    return oracle.from_f32((x * inv) * oracle.to_f32(g_bits, tag), tag)


@pytest.mark.parametrize("tdt,tol", [(torch.float16, 1e-3), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("M,K,widths", [(8, 4096, (4096, 4096, 4096)), (3, 2048, (72, 136)), (13, 4096, (264,)), (1, 4096, (520, 8)),
                                        (20, 4096, (136, 136)), (4, 1024, (64, 64)), (8, 8192, (1024, 136, 136)), (16, 5120, (264, 72)),
                                        (2, 6144, (2048,))])
def test_mm_multi_with_rms_norm_against_oracle(ops, tdt, tol, M, K, widths):
    """rms_norm -> several products in one launch (q, k, v after the first norm of a decoder layer): against the oracle's
    product of the numpy-normalized activations, and against the unfused sequence on the device.  K = 1024 is a shape
    the fused kernel is not built for: the wrapper normalizes with tensor ops."""
    rng = np.random.default_rng(M * 17 + K + len(widths))
    tag = "f16" if tdt == torch.float16 else "bf16"
    cases = [_fused_case(rng, M, n, K, tdt) for n in widths]
    x = (cases[0][2] * 3.0 + 0.5).to(tdt).to(DEV)    # not unit variance, not zero mean
    g = torch.from_numpy(rng.uniform(0.5, 1.5, K).astype(np.float32)).to(tdt).to(DEV)
    packed = [ops._convert_weight_to_int4pack(torch.from_numpy(c).to(DEV), 2) for c, _, _ in cases]
    szs = [sz.to(DEV) for _, sz, _ in cases]
    got = ops.int4pack_mm_multi(x, packed, 128, szs, norm_weight=g, eps=1e-5)
    xn_dev = ops.rms_norm(x, g, 1e-5)
    xn = _rms_norm_bits(host(x), host(g), tag, 1e-5)
    # the normalized activations themselves: device composite against numpy, at most one rounding apart
    assert_close_norm(xn_dev.float().cpu().numpy(), oracle.to_f32(xn, tag), 2.0 ** -10 if tag == "f16" else 2.0 ** -7)
    for (codes, sz, _), p, szd, y, n in zip(cases, packed, szs, got, widths):
        assert tuple(y.shape) == (M, n) and y.dtype == tdt
        assert_close_norm(y.float().cpu().numpy(), ops._weight_int4pack_mm(xn_dev, p, 128, szd).float().cpu().numpy(), 2 * tol)
        tiles = _tile_subset(rng, n // 8, 32)
        cols = (tiles[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
        want = oracle.to_f32(oracle.int4_mm_tc(xn, tag, oracle.int4_pack_tc(codes[cols], 2), host(sz)[:, cols], 128), tag)
        assert_close_norm(y.float().cpu().numpy()[:, cols], want, 2 * tol)


@pytest.mark.parametrize("tdt,tol", [(torch.float16, 1e-3), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("K,widths", [(4096, (264, 136)), (2048, (520,)), (8192, (136,))])
def test_mm_multi_with_rms_norm_row_magnitudes(ops, tdt, tol, K, widths):
    """Rows from 1e-4 to 1e4 in one batch and norm weights from 0.02 to 30: the fused kernel rounds x g before the row's
    factor is known, so in fp16 it has to scale both (x g reaches 3e5 here, and 2e-6 at the other end).  Every row is
    held to the tolerance on its own, against the oracle's product of the normalized activations
    (tensorplay/nn/functional.py:2350-2372: (x inv) g in float32, one rounding)."""
    rng = np.random.default_rng(K + len(widths))
    tag = "f16" if tdt == torch.float16 else "bf16"
    scales = np.array([1e-4, 1e-3, 1.0, 30.0, 1e3, 3e3, 1e4, 0.05], dtype=np.float32)
    M = len(scales)
    cases = [_fused_case(rng, M, n, K, tdt) for n in widths]
    x = (cases[0][2].float() * torch.from_numpy(scales)[:, None]).to(tdt).to(DEV)
    g_np = rng.uniform(0.5, 1.5, K).astype(np.float32) * rng.choice(np.array([0.04, 1.0, 20.0], dtype=np.float32), K)
    g = torch.from_numpy(g_np).to(tdt).to(DEV)
    assert torch.isfinite(x).all()
    packed = [ops._convert_weight_to_int4pack(torch.from_numpy(c).to(DEV), 2) for c, _, _ in cases]
    szs = [sz.to(DEV) for _, sz, _ in cases]
    got = ops.int4pack_mm_multi(x, packed, 128, szs, norm_weight=g, eps=1e-5)
    xn = _rms_norm_bits(host(x), host(g), tag, 1e-5)
    for (codes, sz, _), y, n in zip(cases, got, widths):
        y = y.float().cpu().numpy()
        assert np.isfinite(y).all()
        want = oracle.to_f32(oracle.int4_mm_tc(xn, tag, oracle.int4_pack_tc(codes, 2), host(sz), 128), tag)
        for r in range(M):
            assert_close_norm(y[r:r + 1], want[r:r + 1], 2 * tol, "row of magnitude %g" % scales[r])


@pytest.mark.parametrize("tdt,tol", [(torch.float16, 2e-3), (torch.bfloat16, 1.6e-2)])
@pytest.mark.parametrize("M,N,K", [(8, 11008, 4096), (2, 72, 4096), (5, 136, 2048), (12, 200, 4096), (3, 64, 512)])
def test_mm_swiglu_with_rms_norm_against_oracle(ops, tdt, tol, M, N, K):
    """rms_norm -> gate / up -> silu_mul in one launch (the MLP front of a decoder layer)."""
    rng = np.random.default_rng(M * 29 + N)
    tag = "f16" if tdt == torch.float16 else "bf16"
    cg, szg, x = _fused_case(rng, M, N, K, tdt)
    cu, szu, _ = _fused_case(rng, M, N, K, tdt)
    x = (x * 2.0 - 0.25).to(tdt).to(DEV)
    g = torch.from_numpy(rng.uniform(0.5, 1.5, K).astype(np.float32)).to(tdt).to(DEV)
    pg = ops._convert_weight_to_int4pack(torch.from_numpy(cg).to(DEV), 2)
    pu = ops._convert_weight_to_int4pack(torch.from_numpy(cu).to(DEV), 2)
    got = ops.int4pack_mm_swiglu(x, pg, pu, 128, szg.to(DEV), szu.to(DEV), norm_weight=g, eps=1e-5)
    xn = _rms_norm_bits(host(x), host(g), tag, 1e-5)
    tiles = _tile_subset(rng, N // 8, 32)
    cols = (tiles[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
    og = oracle.to_f32(oracle.int4_mm_tc(xn, tag, oracle.int4_pack_tc(cg[cols], 2), host(szg)[:, cols], 128), tag)
    ou = oracle.to_f32(oracle.int4_mm_tc(xn, tag, oracle.int4_pack_tc(cu[cols], 2), host(szu)[:, cols], 128), tag)
    want = og * (1.0 / (1.0 + np.exp(-og))) * ou
    assert_close_norm(got.float().cpu().numpy()[:, cols], want, 2 * tol)


def test_mm_multi_other_shapes_and_errors(ops):
    rng = np.random.default_rng(6)
    codes = rng.integers(0, 16, (32, 128)).astype(np.int32)
    packed = ops._convert_weight_to_int4pack(torch.from_numpy(codes).to(DEV), 2)
    sz = torch.rand(4, 32, 2, device=DEV).half() * 0.01   # groups of 32: the separate op runs
    x = torch.randn(3, 128, device=DEV).half()
    outs = ops.int4pack_mm_multi(x, [packed, packed], 32, [sz, sz])
    assert torch.equal(outs[0], ops._weight_int4pack_mm(x, packed, 32, sz)) and torch.equal(outs[0], outs[1])
    sz128 = torch.rand(1, 32, 2, device=DEV).half() * 0.01
    five = ops.int4pack_mm_multi(x, [packed] * 5, 128, [sz128] * 5)   # more than four weights: separate ops
    assert len(five) == 5 and torch.equal(five[0], five[4])
    assert ops.int4pack_mm_multi(x[:0], [packed], 128, [sz128])[0].shape == (0, 32)
    with pytest.raises(ValueError):
        ops.int4pack_mm_multi(x, [packed, packed], 128, [sz128])
    with pytest.raises(ValueError):
        ops.int4pack_mm_multi(x, [], 128, [])


def test_fused_entry_points_fall_back_for_other_shapes(ops):
    rng = np.random.default_rng(5)
    codes = rng.integers(0, 16, (32, 128)).astype(np.int32)
    packed = ops._convert_weight_to_int4pack(torch.from_numpy(codes).to(DEV), 2)
    sz = torch.rand(4, 32, 2, device=DEV).half() * 0.01   # groups of 32: not a fused shape
    x = torch.randn(3, 128, device=DEV).half()
    res = torch.randn(3, 32, device=DEV).half()
    assert torch.equal(ops.int4pack_mm_add(x, packed, 32, sz, res), res + ops._weight_int4pack_mm(x, packed, 32, sz))
    out = ops.int4pack_mm_swiglu(x, packed, packed, 32, sz, sz)
    g = ops._weight_int4pack_mm(x, packed, 32, sz).float()
    assert torch.equal(out, (g * torch.sigmoid(g) * g).half())


@pytest.mark.parametrize("K,taken", [(1024, False), (2048, True), (4096, True), (5120, True), (8192, True), (11008, False)])
def test_norm_entry_point_takes_the_shapes_it_names(ops, K, taken):
    """tpq_int4_mm_multi_norm through the C ABI: OK for K = 2048..8192, TPQ_ERR_UNSUPPORTED outside (the wrapper then runs
    the norm and the plain entry), so the oracle comparisons above do exercise the fused kernel at those K."""
    import ctypes
    from tensorplay_amd import _lib
    rng = np.random.default_rng(K)
    n, m = 136, 5
    codes = rng.integers(0, 16, (n, K)).astype(np.int32)
    packed = ops._convert_weight_to_int4pack(torch.from_numpy(codes).to(DEV), 2)
    sz = (torch.rand(K // 128, n, 2, device=DEV) * 0.01).half()
    x = torch.randn(m, K, device=DEV).half()
    g = torch.ones(K, device=DEV).half()
    out = torch.empty(m, n, device=DEV).half()
    ptrs = lambda t: (ctypes.c_void_p * 1)(t.data_ptr())
    widths = (ctypes.c_int64 * 1)(n)
    status = _lib.load().tpq_int4_mm_multi_norm(x.data_ptr(), 1, m, K, g.data_ptr(), 1e-5, 1, ctypes.cast(ptrs(packed), ctypes.c_void_p), 2,
                                                ctypes.cast(widths, ctypes.c_void_p), 128, ctypes.cast(ptrs(sz), ctypes.c_void_p),
                                                ctypes.cast(ptrs(out), ctypes.c_void_p), torch.cuda.current_stream().cuda_stream)
    assert status == (0 if taken else _lib.TPQ_ERR_UNSUPPORTED)
    if taken:
        torch.cuda.synchronize()
        want = ops._weight_int4pack_mm(ops.rms_norm(x, g, 1e-5), packed, 128, sz)
        assert_close_norm(out.float().cpu().numpy(), want.float().cpu().numpy(), 2e-3)


# ---- the decoder layer of the benchmark configuration: seven int4 linears at batch 8 -----------------------------------

class _LayerWeight:
    """One int4 g=128 weight of the layer on the device, plus what the oracle needs for a subset of its channels."""

    def __init__(self, ops, rng, n, k):
        w = rng.normal(0, 0.02, (n, k)).astype(np.float32)
        self.codes, sz = asym_quant(w, 128)
        self.sz_bits = cast_bits(sz, "f16")                       # [K/128, N, 2] fp16 bits
        self.packed = ops._convert_weight_to_int4pack(dev(self.codes), 2)
        self.sz = dev(self.sz_bits, "f16")
        self.n, self.k = n, k
        tiles = _tile_subset(rng, n // 8, 48)                     # 384 channels: the oracle takes well under a second
        self.cols = (tiles[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)

    def oracle_products(self, x_bits):
        """(device formulation rounded to fp16 as float32, exact fp64 sums) on the channel subset."""
        packed = oracle.int4_pack_tc(self.codes[self.cols], 2)
        sz = np.ascontiguousarray(self.sz_bits[:, self.cols])
        ref = oracle.to_f32(oracle.int4_mm_tc(x_bits, "f16", packed, sz, 128, round_w=True), "f16")
        _, y64 = oracle.int4_mm_tc(x_bits, "f16", packed, sz, 128, round_w=False, want_f64=True)
        return ref, y64


def _check_product(got, weight, x_bits, what):
    ref, y64 = weight.oracle_products(x_bits)
    sub = got.float().cpu().numpy()[:, weight.cols]
    assert_close_norm(sub, ref, 1e-2, f"{what} vs reference formulation")
    assert rel_err(sub, y64) < 1e-3, f"{what} vs fp64 sums: {rel_err(sub, y64):.2e}"


def test_decoder_layer_linears_batch8_against_oracle(ops):
    """Llama-style layer, d = 4096, MLP 11008, batch 8, fp16, all seven linears int4 in groups of 128
    (the reference's layer: benchmark/bench_llama_e2e.py:107-144), each through the entry point the layer uses:
    q, k, v in one launch, o and down with the residual added in the epilogue, gate and up with the SwiGLU epilogue,
    and each also through the plain op.  Checked against the oracle on 384 channels per weight: 1e-2 against the
    reference's device formulation, 1e-3 against the fp64 sums."""
    d, inter, M = 4096, 11008, 8
    rng = np.random.default_rng(505)
    print("config 5: building seven int4 weights", flush=True)
    wq, wk, wv, wo = (_LayerWeight(ops, rng, d, d) for _ in range(4))
    wg, wu = _LayerWeight(ops, rng, inter, d), _LayerWeight(ops, rng, inter, d)
    wd = _LayerWeight(ops, rng, d, inter)
    xb = cast_bits(rng.normal(0, 1, (M, d)).astype(np.float32), "f16")       # normed hidden state
    hb = cast_bits(rng.normal(0, 0.3, (M, inter)).astype(np.float32), "f16")  # MLP activations
    rb = cast_bits(rng.normal(0, 1, (M, d)).astype(np.float32), "f16")       # residual stream
    x, h, res = dev(xb, "f16"), dev(hb, "f16"), dev(rb, "f16")

    # q, k, v: one launch
    print("config 5: q, k, v (int4pack_mm_multi)", flush=True)
    qkv = ops.int4pack_mm_multi(x, [wq.packed, wk.packed, wv.packed], 128, [wq.sz, wk.sz, wv.sz])
    for name, w, y in zip("qkv", (wq, wk, wv), qkv):
        assert tuple(y.shape) == (M, d) and y.dtype == torch.float16
        _check_product(y, w, xb, name)
        _check_product(ops._weight_int4pack_mm(x, w.packed, 128, w.sz), w, xb, name + " (plain op)")

    # o and down: residual added in the epilogue, out = T(T(x.W^T) + residual)
    for name, w, inp, inp_bits in (("o", wo, x, xb), ("down", wd, h, hb)):
        print(f"config 5: {name} (int4pack_mm_add, K = {w.k})", flush=True)
        plain = ops._weight_int4pack_mm(inp, w.packed, 128, w.sz)
        _check_product(plain, w, inp_bits, name + " (plain op)")
        got = ops.int4pack_mm_add(inp, w.packed, 128, w.sz, res)
        ref, y64 = w.oracle_products(inp_bits)
        r32 = oracle.to_f32(rb, "f16")[:, w.cols]
        want = oracle.to_f32(cast_bits(ref + r32, "f16"), "f16")              # both roundings of the separate ops
        sub = got.float().cpu().numpy()[:, w.cols]
        assert_close_norm(sub, want, 1e-2, f"{name} + residual vs reference formulation")
        assert rel_err(sub, y64 + r32) < 1e-3, f"{name} + residual vs fp64"
        assert torch.equal(got, (plain + res)), f"{name}: fused epilogue differs from the separate add"

    # gate, up: one launch, silu_mul epilogue
    print("config 5: gate, up (int4pack_mm_swiglu)", flush=True)
    got = ops.int4pack_mm_swiglu(x, wg.packed, wu.packed, 128, wg.sz, wu.sz)
    assert tuple(got.shape) == (M, inter)
    cols = wu.cols = wg.cols   # same channels of both weights
    g_ref, g64 = wg.oracle_products(xb)
    u_ref, u64 = wu.oracle_products(xb)
    want = g_ref * (1.0 / (1.0 + np.exp(-g_ref.astype(np.float64)))) * u_ref   # silu_mul of the two rounded products
    exact = g64 * (1.0 / (1.0 + np.exp(-g64))) * u64
    sub = got.float().cpu().numpy()[:, cols]
    assert_close_norm(sub, want, 1e-2, "swiglu vs reference formulation")
    assert rel_err(sub, exact) < 2e-3, f"swiglu vs fp64: {rel_err(sub, exact):.2e}"  # two fp16 roundings feed a product
    _check_product(ops._weight_int4pack_mm(x, wg.packed, 128, wg.sz), wg, xb, "gate (plain op)")
    _check_product(ops._weight_int4pack_mm(x, wu.packed, 128, wu.sz), wu, xb, "up (plain op)")


# ---- one row on the kernel that deals whole tiles of eight channels to the compute units ---------------------------------

@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("N,K,group", [
    (4096, 256, 128),      # one block per tile: a single wavefront per workgroup
    (2056, 2560, 128),     # ten wavefronts; fewer tiles than workgroups x 2, a last partial group of four tiles
    (16400, 4096, 32),     # 16 wavefronts, nine rounds = two batches, groups of 32 (eight groups per block)
    (4104, 5120, 64),      # two blocks per wavefront (ten wavefronts)
    (2048, 11008, 128),    # three blocks per wavefront, 15 wavefronts, the last with a block past K
    (520, 8192, 128),      # fewer tiles than workgroups: most workgroups idle
    (5120, 13824, 128),    # four blocks per wavefront (14 wavefronts, the last with two blocks past K), several batches of one round
    (1032, 16384, 64),     # four blocks for each of 16 wavefronts, groups of 64
])
def test_mm_one_row_tile_streaming_kernel(ops, kernel_override, dtype, N, K, group):
    """kernel_override("int4_row", 1) pins the one-row kernel for every shape it can take (its default shapes are few and
    large): against the fp64 sums (1e-3 fp16, 1e-2 bf16), the reference's device formulation (1e-2), and the default route."""
    rng = np.random.default_rng(N + K + group)
    codes, sz = asym_quant(rng.normal(0, 0.02, (N, K)).astype(np.float32), group)
    x = rng.normal(0, 1, (1, K)).astype(np.float32)
    xb, szb = cast_bits(x, dtype), cast_bits(sz, dtype)
    packed = oracle.int4_pack_tc(codes, 2)
    args = (dev(xb, dtype), dev(packed), group, dev(szb, dtype))
    default = ops._weight_int4pack_mm(*args).float().cpu().numpy()
    kernel_override("int4_row", 1)
    got = ops._weight_int4pack_mm(*args).float().cpu().numpy()
    tiles = _tile_subset(rng, N // 8, 64)   # the oracle on 512 channels: first and last tile included
    cols = (tiles[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
    sub_packed, sub_sz = oracle.int4_pack_tc(codes[cols], 2), np.ascontiguousarray(szb[:, cols])
    ref_dev = oracle.to_f32(oracle.int4_mm_tc(xb, dtype, sub_packed, sub_sz, group, round_w=True), dtype)
    _, y64 = oracle.int4_mm_tc(xb, dtype, sub_packed, sub_sz, group, round_w=False, want_f64=True)
    assert_close_to_cpu_formulation(got, xb, dtype, codes, szb, group)
    assert_close_norm(got[:, cols], ref_dev, 1.5e-2 if dtype == "bf16" else 1e-2, "row kernel vs the device formulation (secondary)")
    assert rel_err(got[:, cols], y64) < (1e-3 if dtype == "f16" else 1e-2)
    # every channel against the default route (another kernel, another order of the fp32 additions)
    assert rel_err(got, default) < (2e-3 if dtype == "f16" else 1.6e-2)


def test_mm_one_row_down_projection_default_route(ops):
    """11008 -> 4096 at one row: the shape the tile-streaming kernel serves by default."""
    rng = np.random.default_rng(77)
    N, K = 4096, 11008
    codes, sz = asym_quant(rng.normal(0, 0.02, (N, K)).astype(np.float32), 128)
    xb, szb = cast_bits(rng.normal(0, 1, (1, K)).astype(np.float32), "f16"), cast_bits(sz, "f16")
    got = ops._weight_int4pack_mm(dev(xb, "f16"), dev(oracle.int4_pack_tc(codes, 2)), 128, dev(szb, "f16")).float().cpu().numpy()
    tiles = _tile_subset(rng, N // 8, 48)
    cols = (tiles[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
    _, y64 = oracle.int4_mm_tc(xb, "f16", oracle.int4_pack_tc(codes[cols], 2), np.ascontiguousarray(szb[:, cols]), 128,
                               round_w=False, want_f64=True)
    assert rel_err(got[:, cols], y64) < 1e-3


# ---- one row of a wide weight at lengths other than 2048 / 4096 / 6144: the looped form of the column-per-lane kernel ------

@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("N,K", [
    (10304, 2560),    # 20 chunks of 128 k: twelve of the 16 wavefronts take one, four take two
    (10240, 5120),    # 40 chunks
    (10248, 7168),    # 56 chunks; ragged last column group
    (10240, 8192),    # 64 chunks: four per wavefront
    (10240, 10240),   # five
    (10312, 11008),   # 86 chunks
    (10240, 14336),   # seven per wavefront
    (20488, 8192),    # wide and ragged at K = 8192: the tile-streaming kernel in several batches, a last partial tile group
    (8200, 12288),    # K = 12288: three blocks per wavefront
    (20552, 5120),    # column groups whose last round is short: the tile-streaming kernel at K = 5120
])
def test_mm_one_row_wide_weight_other_lengths(ops, dtype, N, K):
    """One row of a wide weight where K / 128 is not 16, 32 or 48 (the looped column-per-lane kernel, or the tile-streaming
    kernel where the library prefers it): against the fp64 sums (1e-3 fp16,
    1e-2 bf16) and the reference's device formulation (1e-2 / 1.5e-2) on a subset of whole tiles that contains the first
    and the last, and every channel against the 2-row call's first row (the matrix-core kernel: another order of sums)."""
    rng = np.random.default_rng(N + K)
    codes, sz = asym_quant(rng.normal(0, 0.02, (N, K)).astype(np.float32), 128)
    x = rng.normal(0, 1, (2, K)).astype(np.float32)
    xb, szb = cast_bits(x, dtype), cast_bits(sz, dtype)
    packed = dev(oracle.int4_pack_tc(codes, 2))
    got = ops._weight_int4pack_mm(dev(xb[:1], dtype), packed, 128, dev(szb, dtype)).float().cpu().numpy()
    two = ops._weight_int4pack_mm(dev(xb, dtype), packed, 128, dev(szb, dtype)).float().cpu().numpy()
    tiles = _tile_subset(rng, N // 8, 48)
    cols = (tiles[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
    sub_packed, sub_sz = oracle.int4_pack_tc(codes[cols], 2), np.ascontiguousarray(szb[:, cols])
    ref_dev = oracle.to_f32(oracle.int4_mm_tc(xb[:1], dtype, sub_packed, sub_sz, 128, round_w=True), dtype)
    _, y64 = oracle.int4_mm_tc(xb[:1], dtype, sub_packed, sub_sz, 128, round_w=False, want_f64=True)
    assert_close_to_cpu_formulation(got, xb[:1], dtype, codes, szb, 128)
    assert_close_norm(got[:, cols], ref_dev, 1.5e-2 if dtype == "bf16" else 1e-2, "one row vs the device formulation (secondary)")
    assert rel_err(got[:, cols], y64) < (1e-3 if dtype == "f16" else 1e-2)
    assert rel_err(got, two[:1]) < (2e-3 if dtype == "f16" else 1.6e-2)
