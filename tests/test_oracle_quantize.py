"""Pins for the oracle's 16-bit float conversions and row-wise quantizer (A1/A2/N7).

The checks are independent restatements: torch's own casts, a vectorised numpy
float32 closed form, torch.round, and invariants of the definition
(reference: p10/include/QuantNativeImpl.h:1162-1187,
test/quantization/test_int8_dyn_act_lowbit.py:90-102).
"""
import zlib

import numpy as np
import pytest
import torch

import oracle
from helpers import bits_of, cast_bits, from_bits


def test_f16_to_f32_all_bit_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.to_f32(bits, "f16")
    want = from_bits(bits, "f16").float().numpy()
    np.testing.assert_array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()


def test_bf16_to_f32_all_bit_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.to_f32(bits, "bf16")
    want = from_bits(bits, "bf16").float().numpy()
    ok = ~np.isnan(want)
    np.testing.assert_array_equal(got.view(np.uint32)[ok], want.view(np.uint32)[ok])


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_f32_to_16bit_matches_torch_rounding(dtype):
    rng = np.random.default_rng(7)
    # random bit patterns cover normals, subnormals, overflow and ties
    raw = rng.integers(0, 2**32, size=400_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    ties = (np.arange(0, 70000, dtype=np.uint32).astype(np.uint32) << 12).view(np.float32)
    small = (rng.normal(size=50_000) * 1e-6).astype(np.float32)
    x = np.concatenate([raw, ties, small, np.float32([0.0, -0.0, 65504, 65519.99, 65520, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-08])])
    x = x[~np.isnan(x)]
    got = oracle.from_f32(x, dtype)
    want = cast_bits(x, dtype)
    np.testing.assert_array_equal(got, want)


def _closed_form(x32, eps, divisor, qmin, qmax):
    absmax = np.abs(x32).max(axis=1).astype(np.float32)
    scale = (np.maximum(absmax, np.float32(eps)) / np.float32(divisor)).astype(np.float32)
    q = np.rint((x32 / scale[:, None]).astype(np.float32))
    return np.clip(q, qmin, qmax).astype(np.int8), scale


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (16, 1024), (7, 2560), (5, 4099)])
def test_int8_rowwise_matches_numpy_closed_form(dtype, shape):
    rng = np.random.default_rng(zlib.crc32(repr((dtype, shape)).encode()))
    x = rng.normal(size=shape).astype(np.float32)
    xb = cast_bits(x, dtype)
    x32 = from_bits(xb, dtype).float().numpy()
    codes, scales = oracle.quantize_int8_rowwise(xb, dtype, 1e-5)
    want_codes, want_scales = _closed_form(x32, 1e-5, 127.0, -127, 127)
    np.testing.assert_array_equal(scales, want_scales)
    np.testing.assert_array_equal(codes, want_codes)


def test_int8_rowwise_matches_torch_round_chain():
    # the reference's eager CPU chain (tensorplay/ao/quantization/bitnet.py:125-135)
    torch.manual_seed(3)
    x = torch.randn(33, 777)
    absmax = x.abs().amax(dim=-1, keepdim=True).clamp(min=1e-5)
    row_scale = absmax / 127.0
    want = (x.float() / row_scale).round().clamp(-127, 127).to(torch.int8)
    codes, scales = oracle.quantize_int8_rowwise(x.numpy(), "f32", 1e-5)
    np.testing.assert_array_equal(codes, want.numpy())
    np.testing.assert_array_equal(scales, row_scale.reshape(-1).numpy())


def test_rowwise_invariants_and_ties():
    x = np.zeros((4, 8), np.float32)
    x[1] = [127, -127, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5]       # scale == 1: ties go to even
    x[2] = [1e-9, -1e-9, 0, 0, 0, 0, 0, 0]                      # below eps
    x[3] = [3, -4, 1, 0, 0, 0, 0, 0]
    codes, scales = oracle.quantize_int8_rowwise(x, "f32", 1e-5)
    assert scales[0] == np.float32(1e-5) / np.float32(127) and not codes[0].any()
    assert scales[1] == 1.0
    assert codes[1].tolist() == [127, -127, 0, 2, 2, 0, -2, -2]
    assert scales[2] == np.float32(1e-5) / np.float32(127)
    assert abs(int(codes[3][1])) == 127 and np.abs(codes).max() <= 127


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_int4_int2_binary_rowwise(dtype):
    rng = np.random.default_rng(11)
    x = rng.normal(size=(6, 16)).astype(np.float32)
    xb = cast_bits(x, dtype)
    x32 = from_bits(xb, dtype).float().numpy()
    c4, s4 = oracle.quantize_int4_rowwise(xb, dtype, 1e-8)
    w4, ws4 = _closed_form(x32, 1e-8, 7.0, -8, 7)
    np.testing.assert_array_equal(c4, w4)
    np.testing.assert_array_equal(s4, ws4)
    # reference test closed forms (test_int8_dyn_act_lowbit.py:90-102)
    c2, s2 = oracle.quantize_int2_rowwise(xb, dtype, 1e-8)
    t = torch.from_numpy(x32)
    scale_ref = t.abs().amax(dim=-1, keepdim=True) / 2.0
    np.testing.assert_array_equal(c2, (t / scale_ref).round().clamp(-2, 1).to(torch.int8).numpy())
    assert np.abs(s2 - scale_ref.reshape(-1).numpy()).max() < 1e-6
    cb, sb = oracle.quantize_binary_rowwise(xb, dtype, 1e-8)
    np.testing.assert_array_equal(cb, np.where(x32 >= 0, 1, -1).astype(np.int8))
    assert np.abs(sb - np.abs(x32).max(axis=1)).max() < 1e-6


def test_empty_rows():
    codes, scales = oracle.quantize_int8_rowwise(np.zeros((0, 8), np.float32))
    assert codes.shape == (0, 8) and scales.shape == (0,)
