"""Packed n-bit weight-only linear (int2 / intx / binary modules of the reference).

CPU: the oracle against numpy restatements of the reference's strided-slice pack / unpack formulas
(tensorplay/ao/quantization/intx_weight_only.py:35-80, binary.py:50-85) and against x @ dq.T in
float64.  GPU: the HIP kernels against the oracle: packing bit-exact, the dense weight bit-exact, the
matmul within the reference tests' own 1e-5 for float32 (test_int2_binary_modules.py:69-89) and 1e-3
of the float64 sums for fp16.
"""
import numpy as np
import pytest
import torch

import oracle


def ref_pack_msb_first(codes, bits):
    """pack_intx: per_byte codes per byte, shift 8 - (i + 1) * bits, zero padded."""
    per_byte = 8 // bits
    rows, cols = codes.shape
    padded = -(-cols // per_byte) * per_byte
    x = np.zeros((rows, padded), np.int32)
    x[:, :cols] = codes
    out = np.zeros((rows, padded // per_byte), np.int32)
    for i in range(per_byte):
        out |= (x[:, i::per_byte] & ((1 << bits) - 1)) << (8 - (i + 1) * bits)
    return out.astype(np.uint8)


def ref_pack_binary(codes):
    """pack_binary: code i of each group of eight in bit i."""
    rows, cols = codes.shape
    padded = -(-cols // 8) * 8
    x = np.zeros((rows, padded), np.uint8)
    x[:, :cols] = codes
    return sum(((x[:, i::8] & 1) << i) for i in range(8)).astype(np.uint8)


def dense_weight(codes, sz, group, bits=None):
    """(code - zero) * scale in float32 with sz [G, N, 2].  The reference's chain is unpack -> .to(int8) -> .to(float32)
    (intx_weight_only.py:80, 119): at 8 bits the uint8 code is reinterpreted as int8 first (128 -> -128)."""
    s = np.repeat(sz[:, :, 0].T, group, axis=1)
    z = np.repeat(sz[:, :, 1].T, group, axis=1)
    c = codes.astype(np.uint8).view(np.int8) if bits == 8 else codes
    return ((c.astype(np.float32) - z) * s).astype(np.float32)


def make_case(rng, bits, N, K, group):
    codes = rng.integers(0, 1 << bits, (N, K)).astype(np.uint8)
    sz = np.stack([rng.uniform(0.01, 0.2, (K // group, N)), rng.integers(0, 1 << bits, (K // group, N)).astype(np.float64)],
                  axis=-1).astype(np.float32)
    return codes, sz


# ---------------------------------------------------------------------------------------------
# oracle (CPU)
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("bits", range(1, 9))
@pytest.mark.parametrize("shape", [(5, 10), (4, 16), (3, 1), (7, 33)])
def test_oracle_pack_matches_reference_formula(bits, shape):
    rng = np.random.default_rng(bits * 100 + shape[1])
    codes = rng.integers(0, 1 << bits, shape).astype(np.uint8)
    packed = oracle.lowbit_pack(codes, bits)
    np.testing.assert_array_equal(packed, ref_pack_msb_first(codes, bits))
    np.testing.assert_array_equal(oracle.lowbit_unpack(packed, bits, shape[1]), codes)


def test_oracle_pack_shapes_of_the_reference_tests():
    rng = np.random.default_rng(0)
    c2 = rng.integers(0, 4, (5, 10)).astype(np.uint8)
    assert oracle.lowbit_pack(c2, 2).shape == (5, 3)        # test_int2_binary_modules.py:57-66
    c1 = rng.integers(0, 2, (4, 10)).astype(np.uint8)
    p1 = oracle.lowbit_pack(c1, 1, lsb_first=True)
    assert p1.shape == (4, 2)                               # :129-137
    np.testing.assert_array_equal(p1, ref_pack_binary(c1))
    np.testing.assert_array_equal(oracle.lowbit_unpack(p1, 1, 10, lsb_first=True), c1)
    # one byte by hand: codes 3,0,2,1 -> 0b11001001
    np.testing.assert_array_equal(oracle.lowbit_pack(np.array([[3, 0, 2, 1]], np.uint8), 2), [[0b11001001]])
    np.testing.assert_array_equal(oracle.lowbit_pack(np.array([[1, 0, 0, 1, 0, 0, 0, 1]], np.uint8), 1, lsb_first=True), [[0b10001001]])


@pytest.mark.parametrize("bits", range(1, 9))
def test_oracle_mm_matches_float64_product(bits):
    rng = np.random.default_rng(40 + bits)
    N, K, group, M = 12, 48, 16, 3
    codes, sz = make_case(rng, bits, N, K, group)
    x = rng.standard_normal((M, K)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    out, y64, dense = oracle.lowbit_mm(x, "f32", ref_pack_msb_first(codes, bits), bits, sz, K, group, bias=bias,
                                       want_f64=True, want_dense=True)
    dq = dense_weight(codes, sz, group, bits)
    np.testing.assert_array_equal(dense, dq)
    want = x.astype(np.float64) @ dq.astype(np.float64).T + bias
    np.testing.assert_allclose(y64, want, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-5)


def test_oracle_eight_bit_codes_are_signed_like_the_reference():
    """bits = 8: unpack_intx returns codes.to(int8) and _dequantize_intx converts that to float, so bytes of 128 and
    more dequantize as (byte - 256 - zero) * scale.  Hand-computed: bytes 0, 127, 128, 200, 255 with zero 3, scale 0.5."""
    packed = np.array([[0, 127, 128, 200, 255, 1, 2, 3]], np.uint8)   # bits = 8: the packed bytes are the codes
    sz = np.array([[[0.5, 3.0]]], np.float32)
    x = np.eye(8, dtype=np.float32)
    out, dense = oracle.lowbit_mm(x, "f32", packed, 8, sz, 8, 8, want_dense=True)
    want = np.array([[-1.5, 62.0, -65.5, -29.5, -2.0, -1.0, -0.5, 0.0]], np.float32)
    np.testing.assert_array_equal(dense, want)
    np.testing.assert_array_equal(out, want.T)
    # and through the numpy restatement of the reference's chain on random bytes
    rng = np.random.default_rng(8)
    codes, sz = make_case(rng, 8, 6, 32, 16)
    assert (codes >= 128).any()
    dense = oracle.lowbit_mm(None, "f32", ref_pack_msb_first(codes, 8), 8, sz, 32, 16, want_dense=True)[1]
    unpacked_int8 = codes.astype(np.uint8).astype(np.int8)            # unpack_intx(...): uint8 fields, then .to(int8)
    s, z = np.repeat(sz[:, :, 0].T, 16, axis=1), np.repeat(sz[:, :, 1].T, 16, axis=1)
    np.testing.assert_array_equal(dense, (unpacked_int8.astype(np.float32) - z) * s)


def test_oracle_binary_is_the_sign_times_scale():
    rng = np.random.default_rng(7)
    N, K = 6, 20
    bits01 = rng.integers(0, 2, (N, K)).astype(np.uint8)
    scale = rng.uniform(0.1, 1.0, (N, 1)).astype(np.float32)
    sz = np.stack([2 * scale[:, 0], np.full(N, 0.5, np.float32)], axis=-1)[None]
    dense = oracle.lowbit_mm(None, "f32", ref_pack_binary(bits01), 1, sz, K, K, lsb_first=True, want_dense=True)[1]
    np.testing.assert_array_equal(dense, (bits01.astype(np.float32) * 2 - 1) * scale)   # binary.py:92-94


# ---------------------------------------------------------------------------------------------
# HIP against the oracle (GPU)
# ---------------------------------------------------------------------------------------------

DEV = "cuda:0"


def rel_err(got, want):
    return float(np.abs(got.astype(np.float64) - want).max() / max(np.abs(want).max(), 1e-30))


@pytest.mark.gpu
@pytest.mark.parametrize("bits", range(1, 9))
@pytest.mark.parametrize("shape", [(5, 10), (64, 256), (3, 1), (130, 77)])
def test_gpu_pack_unpack_bit_exact(bits, shape):
    from tensorplay_amd import ops
    rng = np.random.default_rng(bits + shape[1])
    codes = rng.integers(0, 1 << bits, shape).astype(np.uint8)
    for lsb in ((False, True) if bits == 1 else (False,)):
        packed = ops.pack_lowbit(torch.from_numpy(codes).to(DEV), bits, lsb_first=lsb)
        np.testing.assert_array_equal(packed.cpu().numpy(), oracle.lowbit_pack(codes, bits, lsb_first=lsb))
        back = ops.unpack_lowbit(packed, bits, shape[1], lsb_first=lsb)
        np.testing.assert_array_equal(back.cpu().numpy(), codes)


@pytest.mark.gpu
@pytest.mark.parametrize("bits", range(1, 9))
@pytest.mark.parametrize("N,K,group,M", [(32, 16, 8, 3), (10, 48, 16, 9), (7, 33, 11, 1)])
def test_gpu_mm_float32_small_shapes(bits, N, K, group, M):
    """The shapes of the reference's module tests (K=16, N=32, B=3, groupsize 8) and odd ones: plain kernel."""
    from tensorplay_amd import ops
    rng = np.random.default_rng(bits * 7 + K)
    codes, sz = make_case(rng, bits, N, K, group)
    x = rng.standard_normal((M, K)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    packed = oracle.lowbit_pack(codes, bits)
    want = oracle.lowbit_mm(x, "f32", packed, bits, sz, K, group, bias=bias, want_f64=True)[1]
    got = ops._lowbit_mm(torch.from_numpy(x).to(DEV), torch.from_numpy(packed).to(DEV), bits, K, torch.from_numpy(sz).to(DEV),
                         torch.from_numpy(bias).to(DEV))
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("bits,lsb", [(b, False) for b in range(1, 9)] + [(1, True)])
@pytest.mark.parametrize("N,K,group,M", [(64, 256, 128, 1), (36, 512, 256, 3), (48, 1024, 128, 16), (16, 384, 128, 17), (20, 128, 128, 2)])
@pytest.mark.parametrize("tdt,tag,tol", [(torch.float16, "f16", 1e-3), (torch.bfloat16, "bf16", 8e-3)])  # output rounding 5e-4 / 4e-3
def test_gpu_mm_decode_kernel(bits, lsb, N, K, group, M, tdt, tag, tol):
    from tensorplay_amd import ops
    rng = np.random.default_rng(bits * 13 + K + M)
    codes, sz = make_case(rng, bits, N, K, group)
    x16 = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(tdt)
    bias = rng.standard_normal(N).astype(np.float32) if M % 2 else None
    packed = oracle.lowbit_pack(codes, bits, lsb_first=lsb)
    want = oracle.lowbit_mm(x16.view(torch.int16).numpy().view(np.uint16), tag, packed, bits, sz, K, group, bias=bias,
                            lsb_first=lsb, want_f64=True)[1]
    got = ops._lowbit_mm(x16.to(DEV), torch.from_numpy(packed).to(DEV), bits, K, torch.from_numpy(sz).to(DEV),
                         None if bias is None else torch.from_numpy(bias).to(DEV), lsb_first=lsb)
    assert got.dtype == tdt and got.shape == (M, N)
    assert rel_err(got.float().cpu().numpy(), want) < tol


@pytest.mark.gpu
@pytest.mark.parametrize("bits,lsb", [(1, True), (2, False), (3, False), (4, False), (8, False)])
@pytest.mark.parametrize("N,K,group,M", [(4104, 2048, 128, 5), (10248, 2048, 128, 9), (10244, 4096, 128, 16), (4100, 2048, 64, 2), (8200, 2048, 256, 20)])
@pytest.mark.parametrize("tdt,tag,tol", [(torch.float16, "f16", 1e-3), (torch.bfloat16, "bf16", 8e-3)])
def test_gpu_mm_decode_kernel_wide_weights(bits, lsb, N, K, group, M, tdt, tag, tol):
    """Wide weights with 16 steps of K and more: two and three blocks of 16 channels per workgroup share the activations
    of a step; channel counts that leave the last workgroup with a partial block and with whole blocks missing, 2..20
    rows (one and four loads of activations per step, a second slab of rows), with a bias."""
    from tensorplay_amd import ops
    rng = np.random.default_rng(bits * 17 + N + M)
    codes, sz = make_case(rng, bits, N, K, group)
    x16 = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(tdt)
    bias = rng.standard_normal(N).astype(np.float32)
    packed = oracle.lowbit_pack(codes, bits, lsb_first=lsb)
    want = oracle.lowbit_mm(x16.view(torch.int16).numpy().view(np.uint16), tag, packed, bits, sz, K, group, bias=bias,
                            lsb_first=lsb, want_f64=True)[1]
    got = ops._lowbit_mm(x16.to(DEV), torch.from_numpy(packed).to(DEV), bits, K, torch.from_numpy(sz).to(DEV),
                         torch.from_numpy(bias).to(DEV), lsb_first=lsb)
    assert got.dtype == tdt and got.shape == (M, N)
    assert rel_err(got.float().cpu().numpy(), want) < tol


@pytest.mark.gpu
@pytest.mark.parametrize("bits,lsb", [(1, False), (1, True), (2, False), (2, True), (4, False), (4, True), (8, False)])
@pytest.mark.parametrize("N,K,group", [(10, 4096, 128), (7, 8192, 64), (130, 4160, 32), (5, 20480, 1024), (1, 64, 64), (36, 11008, 128),
                                       # rows of 64 KB and 128 KB: the activation row in LDS beyond the default limit (1 and 2 bits)
                                       (3, 32768, 256), (2, 65536, 4096)])
@pytest.mark.parametrize("tdt,tag,tol", [(torch.float16, "f16", 1e-3), (torch.bfloat16, "bf16", 8e-3)])
def test_gpu_mm_one_row_kernel(bits, lsb, N, K, group, tdt, tag, tol, kernel_override):
    """One activation row on the kernel that streams the packed rows: several passes per channel, a last segment
    past K, ragged N, both bit orders, both workgroup sizes (by K), groups of one segment and of many, with a bias.
    kernel_override("lowbit_row", 1) pins the kernel (it is also the default for these shapes) where the row kernel
    is built for the group size; the other cases run on the kernel the library picks."""
    from tensorplay_amd import ops
    if group % {1: 64, 2: 64, 4: 32, 8: 16}[bits] == 0:
        kernel_override("lowbit_row", 1)  # groups shorter than a lane's segment: the library's own choice, same check
    rng = np.random.default_rng(bits * 17 + K + N)
    codes, sz = make_case(rng, bits, N, K, group)
    x16 = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).to(tdt)
    bias = rng.standard_normal(N).astype(np.float32) if N % 2 else None
    packed = oracle.lowbit_pack(codes, bits, lsb_first=lsb)
    want = oracle.lowbit_mm(x16.view(torch.int16).numpy().view(np.uint16), tag, packed, bits, sz, K, group, bias=bias,
                            lsb_first=lsb, want_f64=True)[1]
    got = ops._lowbit_mm(x16.to(DEV), torch.from_numpy(packed).to(DEV), bits, K, torch.from_numpy(sz).to(DEV),
                         None if bias is None else torch.from_numpy(bias).to(DEV), lsb_first=lsb)
    assert got.shape == (1, N)
    assert rel_err(got.float().cpu().numpy(), want) < tol


@pytest.mark.gpu
@pytest.mark.parametrize("bits,N,K", [(1, 8198, 4160), (2, 8198, 4160), (4, 8198, 4160), (1, 8198, 8192), (2, 4100, 16448)])
def test_gpu_mm_one_row_default_route_large_weight(bits, N, K):
    """Model-sized weights with a ragged N and a last segment past K, on the default route: four channels per wavefront,
    and eight for 1 and 2 bits from 2^26 codes on (the last two shapes)."""
    from tensorplay_amd import ops
    rng = np.random.default_rng(90 + bits)
    group = 32 if bits == 4 else 64
    codes, sz = make_case(rng, bits, N, K, group)
    x16 = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).half()
    packed = oracle.lowbit_pack(codes, bits)
    want = x16.double().numpy() @ dense_weight(codes, sz, group, bits).astype(np.float64).T
    got = ops._lowbit_mm(x16.to(DEV), torch.from_numpy(packed).to(DEV), bits, K, torch.from_numpy(sz).to(DEV))
    assert rel_err(got.float().cpu().numpy(), want) < 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("tdtype", [torch.bfloat16, torch.float16])
def test_gpu_mm_other_routes(tdtype):
    """bf16 activations, and N % 4 != 0 / groups that the decode kernel does not take: plain kernel."""
    from tensorplay_amd import ops
    rng = np.random.default_rng(5)
    N, K, group, M = 18, 256, 64, 5
    codes, sz = make_case(rng, 2, N, K, group)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(tdtype)
    packed = oracle.lowbit_pack(codes, 2)
    want = x.double().numpy() @ dense_weight(codes, sz, group).astype(np.float64).T
    got = ops._lowbit_mm(x.to(DEV), torch.from_numpy(packed).to(DEV), 2, K, torch.from_numpy(sz).to(DEV))
    assert rel_err(got.float().cpu().numpy(), want) < (1e-2 if tdtype == torch.bfloat16 else 1e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("bits", [1, 2, 3, 4, 8])
def test_gpu_dequantize_bit_exact_and_many_rows(bits):
    from tensorplay_amd import ops
    rng = np.random.default_rng(60 + bits)
    N, K, group = 40, 256, 128
    codes, sz = make_case(rng, bits, N, K, group)
    packed = torch.from_numpy(oracle.lowbit_pack(codes, bits)).to(DEV)
    dense = ops._lowbit_dequantize(packed, bits, K, torch.from_numpy(sz).to(DEV), torch.float32)
    np.testing.assert_array_equal(dense.cpu().numpy(), dense_weight(codes, sz, group, bits))
    dense16 = ops._lowbit_dequantize(packed, bits, K, torch.from_numpy(sz).to(DEV), torch.float16)
    np.testing.assert_array_equal(dense16.cpu().numpy(), dense_weight(codes, sz, group, bits).astype(np.float16))
    M = ops.LOWBIT_PREFILL_ROWS_SMALL + 5   # dequantise + one dense GEMM
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32))
    got = ops._lowbit_mm(x.to(DEV), packed, bits, K, torch.from_numpy(sz).to(DEV))
    want = x.double().numpy() @ dense_weight(codes, sz, group, bits).astype(np.float64).T
    assert rel_err(got.cpu().numpy(), want) < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("lsb_first", [False, True])
@pytest.mark.parametrize("bits", range(1, 9))
@pytest.mark.parametrize("N,K,group", [(24, 1024, 64), (7, 2056, 8), (5, 132, 66)])
def test_gpu_dequantize_vector_and_plain_kernels(bits, lsb_first, N, K, group):
    """Dense weight in float32 / float16 / bfloat16, bit for bit: rows taken eight k per thread (K and group
    multiples of 8, several groups and threads per row) and the per-element kernel (K = 132)."""
    from tensorplay_amd import ops
    rng = np.random.default_rng(bits * 7 + K + int(lsb_first))
    codes, sz = make_case(rng, bits, N, K, group)
    packed = torch.from_numpy(oracle.lowbit_pack(codes, bits, lsb_first)).to(DEV)
    want = torch.from_numpy(dense_weight(codes, sz, group, bits))
    szd = torch.from_numpy(sz).to(DEV)
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        got = ops._lowbit_dequantize(packed, bits, K, szd, dtype, lsb_first)
        assert torch.equal(got.cpu(), want.to(dtype)), (bits, lsb_first, dtype)


@pytest.mark.gpu
def test_gpu_modules_follow_the_reference_tests():
    """from_float + forward against the manual group-wise formula, as test_int2_binary_modules.py:69-89, 140-155."""
    import torch.nn as nn
    from tensorplay_amd.ao import quantization as q
    torch.manual_seed(0)
    x = torch.randn(3, 16, device=DEV)
    lin = nn.Linear(16, 32, bias=False).to(DEV)

    mod = q.WeightOnlyInt2Linear.from_float(lin, groupsize=8)
    assert mod.weight.dtype == torch.uint8 and mod.weight.shape == (32, 4) and mod.scales_and_zeros.shape == (2, 32, 2)
    scale = mod.scales_and_zeros[..., 0].t().contiguous().repeat_interleave(8, dim=-1)
    zero = mod.scales_and_zeros[..., 1].t().contiguous().repeat_interleave(8, dim=-1)
    dq = (q.unpack_int2(mod.weight, 16).float() - zero) * scale
    torch.testing.assert_close(mod(x), x @ dq.T, atol=1e-5, rtol=1e-5)
    assert set(dq.div(scale).round().unique().tolist()) <= {-2.0, -1.0, 0.0, 1.0}

    modb = q.WeightOnlyBinaryLinear.from_float(lin)
    assert modb.weight.shape == (32, 2) and modb.scale.shape == (32, 1)
    dqb = (q.unpack_binary(modb.weight, 16).float() * 2.0 - 1.0) * modb.scale
    torch.testing.assert_close(modb(x), x @ dqb.T, atol=1e-5, rtol=1e-5)
    assert float((dqb.abs() - modb.scale).abs().max()) < 1e-5

    for bits in (1, 3, 4, 8):
        modx = q.WeightOnlyIntxLinear.from_float(nn.Linear(16, 32, bias=True).to(DEV), bits=bits, groupsize=8)
        s = modx.scales_and_zeros[..., 0].t().contiguous().repeat_interleave(8, dim=-1)
        z = modx.scales_and_zeros[..., 1].t().contiguous().repeat_interleave(8, dim=-1)
        codes = q.unpack_intx(modx.weight, bits, 16).float()   # int8, as the reference dequantizes it (8 bits wrap)
        torch.testing.assert_close(modx(x), x @ ((codes - z) * s).T + modx.bias, atol=1e-5, rtol=1e-5)

    model = nn.Sequential(nn.Linear(16, 32), nn.ReLU(), nn.Linear(32, 8)).to(DEV)
    qmodel = q.quantize_(model, q.int2_weight_only(groupsize=8))
    assert isinstance(qmodel[0], q.WeightOnlyInt2Linear) and isinstance(qmodel[2], q.WeightOnlyInt2Linear)
    assert qmodel(x).shape == (3, 8)
    assert isinstance(q.quantize_binary_weight_only(nn.Sequential(nn.Linear(16, 16)).to(DEV))[0], q.WeightOnlyBinaryLinear)
    assert isinstance(q.quantize_intx_weight_only(nn.Sequential(nn.Linear(16, 16)).to(DEV), bits=3, groupsize=8)[0], q.WeightOnlyIntxLinear)


@pytest.mark.gpu
def test_gpu_full_size_int2_decode_linearity():
    """4096 -> 11008 at 2 bits, fp16, one row: the sum of two activation vectors maps to the sum of the outputs
    (up to fp16 rounding), and a slice of channels matches the oracle."""
    from tensorplay_amd import ops
    rng = np.random.default_rng(77)
    N, K, group = 11008, 4096, 128
    codes, sz = make_case(rng, 2, N, K, group)
    sz[..., 0] *= 0.1
    packed = oracle.lowbit_pack(codes, 2)
    xa = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).half()
    xb = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).half()
    args = (torch.from_numpy(packed).to(DEV), 2, K, torch.from_numpy(sz).to(DEV))
    ya, yb = ops._lowbit_mm(xa.to(DEV), *args).float(), ops._lowbit_mm(xb.to(DEV), *args).float()
    yab = ops._lowbit_mm((xa.float() + xb.float()).half().to(DEV), *args).float()
    assert float((yab - (ya + yb)).abs().max() / (ya + yb).abs().max()) < 5e-3
    rows = slice(5000, 5064)
    want = oracle.lowbit_mm(xa.view(torch.int16).numpy().view(np.uint16), "f16", packed[rows], 2, sz[:, rows], K, group, want_f64=True)[1]
    assert rel_err(ya[:, rows].cpu().numpy(), want) < 1e-3


@pytest.mark.gpu
def test_gpu_from_float_quantizes_in_the_weight_dtype():
    """from_float of the int2 / intx / binary modules quantizes the weight in its own dtype, as the reference does
    (int2_weight_only.py:207, intx_weight_only.py:204-206, binary.py:151): for a float16 weight the division and the
    rounding happen in float16, which picks other codes at ties than a float32 evaluation would.  The stored
    parameters are the float16 values widened to float32."""
    import torch.nn as nn
    from tensorplay_amd.ao import quantization as q
    torch.manual_seed(3)
    lin = nn.Linear(64, 24, bias=False).to(DEV).half()
    w = lin.weight.detach()

    wg = w.reshape(24, 2, 32)
    # intx, 3 bits: the reference's formulas (intx_weight_only.py:97-107) in float16
    lo, hi = wg.min(-1).values, wg.max(-1).values
    scale = ((hi - lo) / 7.0).clamp(min=1e-8)
    zero = (-lo / scale).round().clamp(0, 7)
    codes = ((wg - lo.unsqueeze(-1)) / scale.unsqueeze(-1)).round().clamp(0, 7).to(torch.uint8).reshape(24, 64)
    mod = q.WeightOnlyIntxLinear.from_float(lin, bits=3, groupsize=32)
    assert torch.equal(q.unpack_intx(mod.weight, 3, 64).view(torch.uint8), codes)
    assert mod.scales_and_zeros.dtype == torch.float32
    assert torch.equal(mod.scales_and_zeros[..., 0].t(), scale.float()) and torch.equal(mod.scales_and_zeros[..., 1].t(), zero.float())

    # int2 (int2_weight_only.py:52-60) in float16
    s2 = (wg.abs().amax(-1) / 2.0).clamp(min=1e-8)
    c2 = ((wg / s2.unsqueeze(-1)).round() + 2.0).clamp(0, 3).to(torch.uint8).reshape(24, 64)
    mod2 = q.WeightOnlyInt2Linear.from_float(lin, groupsize=32)
    assert torch.equal(q.unpack_int2(mod2.weight, 64), c2)
    assert torch.equal(mod2.scales_and_zeros[..., 0].t(), s2.float())

    # binary (binary.py:36-47): per-row mean of |w| in float16
    modb = q.WeightOnlyBinaryLinear.from_float(lin)
    assert torch.equal(modb.scale, w.abs().mean(dim=-1, keepdim=True).clamp(min=1e-8).float())
    assert torch.equal(q.unpack_binary(modb.weight, 64), (w >= 0).to(torch.uint8))
