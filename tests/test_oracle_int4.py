"""Pins for the oracle's int4 layouts and matmuls (A6, A6', A7, A7', A8).

* CPU layout / CPU matmul: byte equality and value equality with PyTorch's CPU
  library ops, the same comparison the reference's own test makes
  (test/quantization/test_native_operator_families.py:579-599).
* Device layout: no CPU library twin exists.  It is pinned by the pack
  following the pack kernels (p10/src/backend/cuda/QuantGemmKernels.cu:322-330,
  838-877) and the unpack following the dequantize kernel (:1170-1202) being
  inverses of each other, plus a direct nibble formula written here.
* Device matmul: closed form (code-8)*scale+zero against an fp64 product, the
  CPU kernel on the same codes, and the reference's symmetric-quantizer check
  (test/quantization/test_int4_modules.py:26-67).
"""
import numpy as np
import pytest
import torch

import oracle
from helpers import TORCH_DT, bits_of, cast_bits, from_bits, rel_err


@pytest.mark.parametrize("channels", [16, 32, 48, 64, 80, 128, 256])
@pytest.mark.parametrize("group", [32, 64, 128, 256])
def test_cpu_layout_bytes_equal_torch(channels, group):
    rng = np.random.default_rng(124)
    features = group * 2
    codes = rng.integers(0, 16, size=(channels, features), dtype="int32")
    want = torch._convert_weight_to_int4pack_for_cpu(torch.tensor(codes), 2).numpy()
    np.testing.assert_array_equal(oracle.int4_pack_cpu(codes, 64, True), want)


def test_cpu_layout_plain_tier_pairs_adjacent_columns():
    codes = np.arange(32 * 4, dtype=np.int32).reshape(32, 4) % 16
    got = oracle.int4_pack_cpu(codes, 32, False)
    for f in range(4):
        for lane in range(16):
            assert got.reshape(-1)[f * 16 + lane] == (codes[2 * lane, f] | (codes[2 * lane + 1, f] << 4))


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("channels,group,rows", [(16, 32, 1), (80, 64, 5), (128, 128, 8), (256, 256, 33), (64, 32, 16)])
def test_cpu_mm_equals_torch_cpu_op(dtype, channels, group, rows):
    rng = np.random.default_rng(124)
    features = group * 2
    codes = rng.integers(0, 16, size=(channels, features), dtype="int32")
    packed = torch._convert_weight_to_int4pack_for_cpu(torch.tensor(codes), 2)
    data = rng.normal(0, 0.2, size=(rows, features)).astype("float32")
    params = rng.uniform(-0.05, 0.05, size=(2, channels, 2)).astype("float32")
    x = torch.tensor(data).to(TORCH_DT[dtype])
    p = torch.tensor(params).to(TORCH_DT[dtype])
    want = torch._weight_int4pack_mm_for_cpu(x, packed, group, p)
    got = oracle.int4_mm_cpu(bits_of(x), dtype, packed.numpy(), bits_of(p), group)
    np.testing.assert_array_equal(got, bits_of(want))


def _tc_word_formula(codes, inner):
    """Device layout written from its description, independent of the two-stage kernels:
    word(nT, kO, t, i2), n = 8 nT + t//4, k0 = (kO*inner + 2*i2)*16 + 2*(t%4);
    bits[4j..4j+3] = code[n, k0+8j], bits[16+4j..] = code[n, k0+8j+1], j = 0..3."""
    N, K = codes.shape
    n_tiles, k_super = (N + 7) // 8, (K + inner * 16 - 1) // (inner * 16)
    out = np.zeros((n_tiles, k_super, 32, inner // 2), np.uint32)
    for nT in range(n_tiles):
        for kO in range(k_super):
            for t in range(32):
                for i2 in range(inner // 2):
                    n = 8 * nT + t // 4
                    k0 = (kO * inner + 2 * i2) * 16 + 2 * (t % 4)
                    w = 0
                    for j in range(4):
                        for odd in (0, 1):
                            k = k0 + 8 * j + odd
                            c = int(codes[n, k]) & 15 if (n < N and k < K) else 0
                            w |= c << (4 * j + 16 * odd)
                    out[nT, kO, t, i2] = w
    return out.view(np.int32)


@pytest.mark.parametrize("inner", [2, 4, 8])
@pytest.mark.parametrize("shape", [(16, 64), (8, 32), (24, 160), (13, 70), (40, 256)])
def test_tc_layout_matches_direct_formula(inner, shape):
    rng = np.random.default_rng(shape[0] * 1000 + shape[1] + inner)
    codes = rng.integers(0, 16, size=shape, dtype="int32")
    np.testing.assert_array_equal(oracle.int4_pack_tc(codes, inner), _tc_word_formula(codes, inner))


@pytest.mark.parametrize("shape", [(16, 64), (8, 32), (24, 160), (13, 70), (64, 4096), (11008 // 8, 128)])
def test_tc_pack_then_dequantize_index_map_round_trips(shape):
    rng = np.random.default_rng(shape[0] + shape[1])
    N, K = shape
    codes = rng.integers(0, 16, size=shape, dtype="int32")
    packed = oracle.int4_pack_tc(codes, 2)
    assert packed.shape == ((N + 7) // 8, (K + 31) // 32, 32, 1)
    back = oracle.int4_unpack_tc(packed, K)
    np.testing.assert_array_equal(back[:N], codes)
    assert not back[N:].any()  # rows beyond N are zero nibbles


def test_tc_stage_one_puts_even_k_in_high_nibble():
    # a single code of 15 at (n=0,k=0) lands in bits 0..3 of word (0,0,0); at k=1 in bits 16..19
    codes = np.zeros((8, 32), np.int32)
    codes[0, 0] = 15
    assert oracle.int4_pack_tc(codes, 2).reshape(-1)[0] == 0xF
    codes[:] = 0
    codes[0, 1] = 15
    assert oracle.int4_pack_tc(codes, 2).reshape(-1)[0] == 0xF0000
    codes[:] = 0
    codes[3, 2 * 2 + 8 * 3 + 1] = 9  # n=3 -> t = 12 + t4, t4 = 2, j = 3, odd
    assert oracle.int4_pack_tc(codes, 2).reshape(-1)[14] == np.int32(np.uint32(9 << 28).view(np.int32))


def _asym_quant(w, group):
    """Asymmetric uint4 group quantizer used by the benchmark configuration:
    s = (max-min)/15, q = clamp(round((w-min)/s), 0, 15), zero = min + 8 s."""
    N, K = w.shape
    wg = w.reshape(N, K // group, group)
    lo, hi = wg.min(-1), wg.max(-1)
    s = np.maximum((hi - lo) / 15.0, 1e-8).astype(np.float32)
    q = np.clip(np.rint((wg - lo[..., None]) / s[..., None]), 0, 15).astype(np.int32).reshape(N, K)
    z = (lo + 8 * s).astype(np.float32)
    return q, np.stack([s.T, z.T], axis=-1)  # [K/g, N, 2]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("M,N,K,group", [(1, 64, 256, 128), (4, 40, 128, 32), (16, 128, 512, 64)])
def test_tc_mm_against_fp64_closed_form_and_cpu_kernel(dtype, M, N, K, group):
    rng = np.random.default_rng(M + N + K)
    w = rng.normal(0, 0.02, (N, K)).astype(np.float32)
    codes, sz = _asym_quant(w, group)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    xb, szb = cast_bits(x, dtype), cast_bits(sz, dtype)
    x32, sz32 = from_bits(xb, dtype).float().numpy().astype(np.float64), from_bits(szb, dtype).float().numpy().astype(np.float64)
    packed = oracle.int4_pack_tc(codes, 2)
    # closed form in fp64 from the rounded parameters
    scale = np.repeat(sz32[:, :, 0].T, group, axis=1)
    zero = np.repeat(sz32[:, :, 1].T, group, axis=1)
    truth = x32 @ ((codes - 8) * scale + zero).T
    y_fp32w, y64 = oracle.int4_mm_tc(xb, dtype, packed, szb, group, round_w=False, want_f64=True)
    assert rel_err(y64, truth) < 1e-6
    tol = {"f32": 1e-6, "f16": 1e-3, "bf16": 8e-3}[dtype]
    assert rel_err(oracle.to_f32(y_fp32w, dtype), truth) < tol
    # device formulation (W rounded to T after each op) stays within the output tolerance
    y_dev = oracle.int4_mm_tc(xb, dtype, packed, szb, group, round_w=True)
    assert rel_err(oracle.to_f32(y_dev, dtype), truth) < {"f32": 1e-6, "f16": 2e-3, "bf16": 1e-2}[dtype]
    # CPU kernel on the same codes (N % 16 == 0 only)
    if N % 16 == 0:
        y_cpu = oracle.int4_mm_cpu(xb, dtype, oracle.int4_pack_cpu(codes), szb, group)
        # fp32 sequential accumulation over K: a few ulp more than the fp64 sum
        assert rel_err(oracle.to_f32(y_cpu, dtype), truth) < max(tol, 5e-6)


def test_symmetric_module_quantizer_reference_check():
    # test_pack_and_mm_matches_reference (test_int4_modules.py:38-67): symmetric codes, zero = 0
    torch.manual_seed(0)
    N, K, B, g = 32, 256, 4, 128
    w, x = torch.randn(N, K), torch.randn(B, K)
    wg = w.reshape(N, K // g, g)
    scale = (wg.abs().amax(dim=-1) / 8.0).clamp(min=1e-8)
    codes = ((wg / scale.unsqueeze(-1)).round().clamp(-8, 7) + 8).to(torch.int32).reshape(N, K)
    sz = torch.stack([scale.t(), torch.zeros_like(scale).t()], dim=-1)
    ref = x @ ((wg / scale.unsqueeze(-1)).round().clamp(-8, 7) * scale.unsqueeze(-1)).reshape(N, K).T
    out = oracle.int4_mm_tc(x.numpy(), "f32", oracle.int4_pack_tc(codes.numpy(), 2), sz.numpy(), g)
    np.testing.assert_allclose(out, ref.numpy(), rtol=1e-2, atol=1e-2)


def test_dequantize_rounds_through_activation_dtype():
    codes = np.full((8, 32), 11, np.int32)
    sz = np.zeros((1, 8, 2), np.float32)
    sz[..., 0], sz[..., 1] = 0.0123, 0.3
    szb = cast_bits(sz, "f16")
    W = oracle.int4_dequantize_tc(oracle.int4_pack_tc(codes), szb, "f16", 32, 32)
    s, z = torch.tensor(sz[0, 0, 0]).half(), torch.tensor(sz[0, 0, 1]).half()
    want = ((torch.tensor(3.0).half() * s).half() + z).half()  # each op rounded to half
    assert (from_bits(W, "f16") == want).all()


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_blocked_baseline_kernel_equals_scalar_kernel(dtype):
    rng = np.random.default_rng(77)
    N, K, g, M = 128, 256, 64, 5
    codes = rng.integers(0, 16, size=(N, K), dtype="int32")
    packed = oracle.int4_pack_cpu(codes)
    x = cast_bits(rng.normal(size=(M, K)).astype(np.float32), dtype)
    sz = cast_bits(rng.uniform(-0.05, 0.05, size=(K // g, N, 2)).astype(np.float32), dtype)
    np.testing.assert_array_equal(oracle.int4_mm_cpu_blocked(x, dtype, packed, sz, g), oracle.int4_mm_cpu(x, dtype, packed, sz, g))
    half = oracle.int4_mm_cpu_blocked(x, dtype, packed, sz, g, blocks=(1, 2))
    np.testing.assert_array_equal(half[:, 64:], oracle.int4_mm_cpu(x, dtype, packed, sz, g)[:, 64:])
