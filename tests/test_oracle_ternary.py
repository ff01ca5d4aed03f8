"""Pins for the oracle's BitNet pieces (A9, A10, A11): the reference tests' literals
(test/quantization/test_native_1bit.py:200-234), the documented bit layout
(tensorplay/ao/quantization/bitnet.py:75-79) and brute force over all byte values."""
import itertools

import numpy as np
import pytest

import oracle


def test_literal_weight_codes():
    w = np.float32([[.4, -.1, .2, -.3], [.0, .6, -.8, .1]])
    scale = oracle.bitnet_scale(w)
    np.testing.assert_allclose(scale, np.abs(w).mean(), rtol=1e-6)
    codes, _ = oracle.quantize_bitnet_weight(w, scale)
    np.testing.assert_array_equal(codes, np.clip(np.round(w / scale), -1, 1))
    assert codes.tolist() == [[1, 0, 1, -1], [0, 1, -1, 0]]


def test_literal_round_trip_2x9():
    codes = np.int8([[1, -1, 0, 1, -1, 0, 0, 1, -1], [0, 1, -1, -1, 1, 0, 1, -1, 0]])
    packed = oracle.pack_ternary(codes)
    assert packed.dtype == np.uint8 and packed.shape == (2, 3)
    np.testing.assert_array_equal(oracle.unpack_ternary(packed, 9), codes)
    # first element in the two most significant bits; -1 -> 0b11, +1 -> 0b01
    assert packed[0, 0] == (0b01 << 6 | 0b11 << 4 | 0b00 << 2 | 0b01)
    assert packed[0, 2] == 0b11 << 6  # zero padded tail


def test_all_ternary_bytes():
    table = np.int8(list(itertools.product([-1, 0, 1], repeat=4)))
    packed = oracle.pack_ternary(table)
    for row, byte in zip(table, packed[:, 0]):
        want = 0
        for q, c in enumerate(row):
            want |= (int(c) & 3) << (6 - 2 * q)
        assert byte == want
    np.testing.assert_array_equal(oracle.unpack_ternary(packed, 4), table)
    # unpack of every byte value is the arithmetic-shift sign extension (0b10 -> -2)
    every = np.arange(256, dtype=np.uint8).reshape(256, 1)
    un = oracle.unpack_ternary(every, 4)
    for b in range(256):
        fields = [(b >> s) & 3 for s in (6, 4, 2, 0)]
        assert un[b].tolist() == [f - 4 if f >= 2 else f for f in fields]


def _manual_bitnet_linear(x, weight, scale=None):
    weight, x = np.asarray(weight, np.float32), np.asarray(x, np.float32)
    if scale is None:
        scale = np.abs(weight).mean()
    codes_w = np.clip(np.round(weight / scale), -1, 1).astype(np.int32)
    absmax = np.maximum(np.abs(x).max(axis=-1, keepdims=True), 1e-5)
    row_scale = absmax / 127.0
    codes_x = np.clip(np.round(x / row_scale), -127, 127).astype(np.int32)
    return (codes_x @ codes_w.T) * row_scale * scale


@pytest.mark.parametrize("shape,N,seed", [((4, 8), 6, 611), ((3, 5), 7, 612), ((6, 2560), 32, 1)])
def test_bitnet_linear_matches_manual_formula(shape, N, seed):
    rng = np.random.default_rng(seed)
    x = rng.normal(size=shape).astype(np.float32)
    w = rng.normal(0, 0.02, size=(N, shape[-1])).astype(np.float32)
    codes, scale = oracle.quantize_bitnet_weight(w)
    packed = oracle.pack_ternary(codes)
    xq, rs = oracle.quantize_int8_rowwise(x, "f32", 1e-5)
    out, acc = oracle.ternary_mm(xq, rs, packed, scale, shape[-1])
    np.testing.assert_array_equal(acc, xq.astype(np.int32) @ codes.astype(np.int32).T)
    np.testing.assert_allclose(out, _manual_bitnet_linear(x, w), rtol=1e-5, atol=1e-5)
