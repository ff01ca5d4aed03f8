"""Block-wise affine quantizer: the oracle against library twins and closed forms (CPU), then the
HIP kernels against the oracle, bit for bit (GPU).

Reference semantics: p10/src/backend/cpu/QuantKernels.cpp:365-455, 579-774; the reference's own
tests compare against torchao's quantize_affine (test/quantization/test_native_1bit.py:24-50,
119-165), which is not installed here: its published formula clamp(round(x * (1/scale)) + zp) is
restated in numpy below.
"""
import ctypes
import zlib

import numpy as np
import pytest
import torch

import oracle

BOUNDS = {"qint8": (-128, 127), "quint8": (0, 255), "qint32": (-2**31, 2**31 - 1),
          "quint4x2": (0, 15), "quint2x4": (0, 3), "quint1x8": (0, 1)}
BITS = {"quint4x2": 4, "quint2x4": 2, "quint1x8": 1}


def blocks_of(shape, block_size):
    """Block index of every element, from coordinates (independent of the oracle's stride walk)."""
    blk = [max(1, min(b, s)) for b, s in zip(block_size, shape)]
    per_dim = [(s + b - 1) // b for s, b in zip(shape, blk)]
    coords = np.indices(shape)
    return np.ravel_multi_index([c // b for c, b in zip(coords, blk)], per_dim), int(np.prod(per_dim))


def closed_form_codes(x, block_size, scales, zeros, lo, hi):
    """clamp(rint(x * (1 / scale)) + zero) per block, in float32, for in-range values."""
    idx, n = blocks_of(x.shape, block_size)
    s = np.broadcast_to(np.asarray(scales, np.float32).reshape(-1), (n,)) if np.size(scales) == 1 else np.asarray(scales, np.float32).reshape(-1)
    inv = np.where(s == 0, np.float32(1), np.float32(1) / s).astype(np.float32)
    pos = np.rint((x.astype(np.float32) * inv[idx]).astype(np.float32))
    if zeros is not None:
        z = np.broadcast_to(np.asarray(zeros, np.float32).reshape(-1), (n,)) if np.size(zeros) == 1 else np.asarray(zeros, np.float32).reshape(-1)
        pos = (pos + z[idx]).astype(np.float32)
    return np.clip(pos.astype(np.int64), lo, hi)


def pack_low_bits_first(codes, bits):
    """Element i in bits (i % pack) * bits of byte i // pack (test_native_1bit.py:43-50 for 1 bit)."""
    pack = 8 // bits
    flat = np.asarray(codes, np.uint8).reshape(-1)
    out = np.zeros((flat.size + pack - 1) // pack, np.uint8)
    for i, c in enumerate(flat):
        out[i // pack] |= np.uint8((int(c) & ((1 << bits) - 1)) << ((i % pack) * bits))
    return out


GRIDS = [
    ((4, 4), (4, 4)), ((4, 4), (1, 4)), ((4, 4), (2, 2)), ((2, 3, 4), (2, 3, 4)), ((2, 3, 4), (1, 1, 4)),
    ((2, 3, 4), (2, 3, 2)),                          # the grids of test_native_1bit.py:119-131
    ((5, 37), (1, 8)), ((7, 64), (1, 32)), ((3, 5, 7), (1, 5, 7)), ((3, 5, 7), (1, 2, 7)), ((6, 10), (4, 3)),
    ((9,), (4,)), ((2, 3, 2, 5), (1, 3, 2, 5)), ((33, 48), (1, 16)),
]


# ---------------------------------------------------------------------------------------------
# oracle (CPU)
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype,tdtype", [("qint8", torch.qint8), ("quint8", torch.quint8), ("qint32", torch.qint32)])
def test_oracle_matches_torch_per_tensor(dtype, tdtype):
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((7, 33)) * 40).astype(np.float32)
    x[0, :8] = np.array([-.5, .5, 1.5, 2.5, 3.5, 4.5, 7.5, 15.5], np.float32) * np.float32(0.37)
    scale, zp = 0.37, 3
    want = torch.quantize_per_tensor(torch.from_numpy(x), scale, zp, tdtype)
    got = oracle.quantize_affine(x, x.shape, [scale], [zp], dtype)
    np.testing.assert_array_equal(got, want.int_repr().numpy())
    back = oracle.dequantize_affine(got, x.shape, x.shape, [scale], [zp], dtype)
    np.testing.assert_array_equal(back, want.dequantize().numpy())


@pytest.mark.parametrize("dtype,tdtype", [("qint8", torch.qint8), ("quint8", torch.quint8)])
def test_oracle_matches_torch_per_channel(dtype, tdtype):
    rng = np.random.default_rng(12)
    x = (rng.standard_normal((9, 50)) * 30).astype(np.float32)
    scales = rng.uniform(0.05, 0.9, 9).astype(np.float32)
    zps = rng.integers(-5, 6, 9) + (100 if dtype == "quint8" else 0)
    want = torch.quantize_per_channel(torch.from_numpy(x), torch.from_numpy(scales).double(), torch.from_numpy(zps), 0, tdtype)
    got = oracle.quantize_affine(x, (1, 50), scales, zps.astype(np.float32), dtype)
    np.testing.assert_array_equal(got, want.int_repr().numpy())
    back = oracle.dequantize_affine(got, x.shape, (1, 50), scales, zps.astype(np.float32), dtype)
    np.testing.assert_array_equal(back, want.dequantize().numpy())


@pytest.mark.parametrize("shape,block", GRIDS)
@pytest.mark.parametrize("dtype", list(BOUNDS))
@pytest.mark.parametrize("with_zero", [False, True])
def test_oracle_matches_closed_form(shape, block, dtype, with_zero):
    rng = np.random.default_rng(zlib.crc32(repr((shape, block, dtype)).encode()))
    lo, hi = BOUNDS[dtype]
    span = min(hi - lo, 255)
    x = rng.uniform(-1.2 * span, 1.2 * span, shape).astype(np.float32)
    _, n = blocks_of(shape, block)
    scales = rng.uniform(0.5, 2.0, n).astype(np.float32)
    zeros = rng.integers(0, 3, n).astype(np.float32) if with_zero else None
    want = closed_form_codes(x, block, scales, zeros, lo, hi)
    got = oracle.quantize_affine(x, block, scales, zeros, dtype)
    if dtype in BITS:
        np.testing.assert_array_equal(got, pack_low_bits_first(want, BITS[dtype]))
    else:
        np.testing.assert_array_equal(got, want)
    back = oracle.dequantize_affine(got, shape, block, scales, zeros, dtype)
    idx, _ = blocks_of(shape, block)
    z = 0 if zeros is None else zeros[idx]
    np.testing.assert_array_equal(back, ((want.astype(np.float32) - z).astype(np.float32) * scales[idx]).astype(np.float32))


@pytest.mark.parametrize("zp,want", [(0, [0, 0, 1, 1, 1, 1, 1, 1]), (1, [1, 1, 1, 1, 1, 1, 1, 1])])
def test_oracle_one_bit_rounding_literals(zp, want):
    """Half-way products round to even before the zero point is added (test_native_1bit.py:57-68)."""
    x = np.array([-.5, .5, 1.5, 2.5, 3.5, 4.5, 7.5, 15.5], np.float32) * np.float32(.25)
    got = oracle.quantize_affine(x, (8,), [.25], [zp], "quint1x8")
    np.testing.assert_array_equal(got, pack_low_bits_first(want, 1))
    back = oracle.dequantize_affine(got, (8,), (8,), [.25], [zp], "quint1x8")
    np.testing.assert_array_equal(back, (np.array(want, np.float32) - zp) * np.float32(.25))


def edge_values():
    return np.array([np.nan, np.inf, -np.inf, 2.0**40, -2.0**40, 2.0**32 + 512, 3e38, -3e38, 2.0**31, -2.0**31,
                     2.0**63, -2.0**63, 0.0, -0.0, 1.5, 2.5], np.float32)


def test_oracle_edge_values_by_hand():
    x = edge_values()
    # byte storage: NaN and anything outside int64 become INT64_MIN -> quant_min; the rest clamps by side
    got = oracle.quantize_affine(x, (16,), [1.0], None, "qint8")
    np.testing.assert_array_equal(got, [-128, -128, -128, 127, -128, 127, -128, -128, 127, -128, -128, -128, 0, 0, 2, 2])
    # packed storage: the int64 is cut to its low 32 bits first: 2^40 -> 0, 2^32 + 512 -> 512 -> 15,
    # INT64_MIN (NaN, inf, 3e38, 2^63) -> 0, -2^63 -> 0, 2^31 -> INT32_MIN -> 0, -2^31 -> 0
    got4 = oracle.quantize_affine(x, (16,), [1.0], None, "quint4x2")
    np.testing.assert_array_equal(got4, pack_low_bits_first([0, 0, 0, 0, 0, 15, 0, 0, 0, 0, 0, 0, 0, 0, 2, 2], 4))
    # a zero scale multiplies by one
    np.testing.assert_array_equal(oracle.quantize_affine(np.array([3.4, -7.6], np.float32), (2,), [0.0], None, "qint8"), [3, -8])


def test_oracle_quant_range_arguments():
    x = np.linspace(-300, 300, 64, dtype=np.float32)
    np.testing.assert_array_equal(oracle.quantize_affine(x, (64,), [1.0], None, "qint8", -127, 127),
                                  np.clip(np.rint(x), -127, 127))
    np.testing.assert_array_equal(oracle.quantize_affine(x, (64,), [1.0], None, "qint8", 0, 0), np.clip(np.rint(x), -128, 127))


# ---------------------------------------------------------------------------------------------
# the C ABI validates before it touches the GPU
# ---------------------------------------------------------------------------------------------

def test_cabi_validation_errors():
    from tensorplay_amd import _lib
    lib = _lib.load()
    arr2 = ctypes.c_int64 * 2
    sizes, blocks = arr2(4, 8), arr2(1, 4)
    p = ctypes.cast(sizes, ctypes.c_void_p)
    b = ctypes.cast(blocks, ctypes.c_void_p)
    # 4 x 2 = 8 blocks: 3 scales is a ValueError
    assert lib.tpq_quantize_affine(None, 0, 2, p, b, None, 3, None, 0, _lib.STORAGE_I8, 0, 0, None, None) == _lib.TPQ_ERR_INVALID_VALUE
    assert "one entry per block" in _lib.last_error()
    assert lib.tpq_quantize_affine(None, 0, 2, p, b, None, 8, None, 5, _lib.STORAGE_I8, 0, 0, None, None) == _lib.TPQ_ERR_INVALID_VALUE
    assert lib.tpq_quantize_affine(None, 0, 2, p, b, None, 8, None, 0, 17, 0, 0, None, None) == _lib.TPQ_ERR_INVALID_TYPE
    assert lib.tpq_quantize_affine(None, 0, 2, p, b, None, 8, None, 0, _lib.STORAGE_U4X2, 0, 16, None, None) == _lib.TPQ_ERR_INVALID_VALUE
    assert "does not fit" in _lib.last_error()
    zero_block = ctypes.cast(arr2(1, 0), ctypes.c_void_p)
    assert lib.tpq_dequantize_affine(None, _lib.STORAGE_I8, 2, p, zero_block, None, 8, None, 0, None, None) == _lib.TPQ_ERR_INVALID_VALUE
    assert "positive" in _lib.last_error()
    # empty tensors succeed without a launch
    empty = ctypes.cast(arr2(0, 8), ctypes.c_void_p)
    assert lib.tpq_quantize_affine(None, 0, 2, empty, b, None, 0, None, 0, _lib.STORAGE_I8, 0, 0, None, None) == _lib.TPQ_OK


# ---------------------------------------------------------------------------------------------
# HIP against the oracle (GPU)
# ---------------------------------------------------------------------------------------------

def _run_gpu(x_t, block, scales, zeros, dtype, qmin=0, qmax=0):
    from tensorplay_amd import ops
    dev = torch.device("cuda:0")
    sc = torch.from_numpy(np.asarray(scales, np.float32)).to(dev)
    zp = None if zeros is None else torch.from_numpy(np.asarray(zeros, np.float32)).to(dev)
    q = ops.quantize_affine(x_t.to(dev), list(block), sc, zp, dtype, qmin, qmax)
    back = ops.dequantize_affine(q, list(block), sc, zp)
    torch.cuda.synchronize()
    raw = q.data if isinstance(q, ops.PackedCodes) else q
    return raw.cpu().numpy(), back.cpu().numpy()


@pytest.mark.gpu
@pytest.mark.parametrize("shape,block", GRIDS + [((64, 256), (1, 128)), ((3, 1000), (1, 1000)), ((130, 48), (1, 48)), ((17, 19), (17, 19)),
                                          ((3, 4), (1, 4)), ((5, 36), (1, 12)), ((1031, 20), (1, 4)), ((2, 1028), (2, 1028))])
@pytest.mark.parametrize("dtype", list(BOUNDS))
def test_gpu_matches_oracle(shape, block, dtype):
    rng = np.random.default_rng(zlib.crc32(repr((shape, block, dtype, 5)).encode()))
    lo, hi = BOUNDS[dtype]
    span = min(hi - lo, 255)
    x = rng.uniform(-1.2 * span, 1.2 * span, shape).astype(np.float32)
    x.reshape(-1)[: min(x.size, 8)] = (np.array([-.5, .5, 1.5, 2.5, 3.5, 4.5, 7.5, 15.5], np.float32) * np.float32(.25))[: min(x.size, 8)]
    _, n = blocks_of(shape, block)
    scales = rng.uniform(0.2, 2.0, n).astype(np.float32)
    scales[0] = .25
    for zeros in (None, rng.integers(0, 3, n).astype(np.float32)):
        want = oracle.quantize_affine(x, block, scales, zeros, dtype)
        want_back = oracle.dequantize_affine(want, shape, block, scales, zeros, dtype)
        got, back = _run_gpu(torch.from_numpy(x), block, scales, zeros, dtype)
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(back, want_back)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", list(BOUNDS))
def test_gpu_scalar_parameters_and_edge_values(dtype):
    x = np.concatenate([edge_values(), np.linspace(-40, 40, 51, dtype=np.float32)]).reshape(1, -1)
    for zeros in (None, [1.0]):
        want = oracle.quantize_affine(x, (1, 16), [0.5], zeros, dtype)
        got, back = _run_gpu(torch.from_numpy(x), (1, 16), [0.5], zeros, dtype)
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(back, oracle.dequantize_affine(want, x.shape, (1, 16), [0.5], zeros, dtype))


@pytest.mark.gpu
@pytest.mark.parametrize("tdtype,name", [(torch.float16, "f16"), (torch.bfloat16, "bf16")])
def test_gpu_sixteen_bit_inputs(tdtype, name):
    """16-bit inputs are widened exactly, as the reference does before its float32 kernel (QuantKernels.cpp:627-629)."""
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(37, 96, generator=g) * 30).to(tdtype)
    scales = np.random.default_rng(4).uniform(0.1, 1.0, 37 * 3).astype(np.float32)
    want = oracle.quantize_affine(x.float().numpy(), (1, 32), scales, None, "qint8", -127, 127)
    got, _ = _run_gpu(x, (1, 32), scales, None, "qint8", -127, 127)
    np.testing.assert_array_equal(got, want)


@pytest.mark.gpu
def test_gpu_full_size_rowwise_codes_and_round_trip():
    """2048 x 4096 activations, one block per row: the step before the int8 GEMM
    (tensorplay/ao/quantization/bitnet.py:127-135 takes this route for large inputs)."""
    g = torch.Generator().manual_seed(8)
    x = torch.randn(2048, 4096, generator=g)
    scales = (x.abs().amax(dim=1).clamp_min(1e-5) / 127.0).numpy()
    want = oracle.quantize_affine(x.numpy(), (1, 4096), scales, None, "qint8", -127, 127)
    got, back = _run_gpu(x, (1, 4096), scales, None, "qint8", -127, 127)
    np.testing.assert_array_equal(got, want)
    assert np.abs(back - x.numpy()).max() <= 0.5 * scales.max() * (1 + 1e-6)


@pytest.mark.gpu
def test_gpu_grouped_weight_four_bit_round_trip():
    """4096 x 4096 weight in groups of 128, unsigned 4-bit with zero point 8."""
    g = torch.Generator().manual_seed(9)
    w = torch.randn(4096, 4096, generator=g)
    grp = w.view(4096, 32, 128)
    scales = (grp.abs().amax(dim=2).clamp_min(1e-6) / 7.0).reshape(-1).numpy()
    zeros = np.full(scales.shape, 8.0, np.float32)
    want = oracle.quantize_affine(w.numpy(), (1, 128), scales, zeros, "quint4x2")
    got, back = _run_gpu(w, (1, 128), scales, zeros, "quint4x2")
    np.testing.assert_array_equal(got, want)
    err = np.abs(back - w.numpy()).reshape(4096, 32, 128).max(axis=2).reshape(-1)
    assert (err <= 0.5 * scales * (1 + 1e-6)).all()


@pytest.mark.gpu
def test_gpu_op_errors():
    from tensorplay_amd import ops
    dev = torch.device("cuda:0")
    x = torch.zeros(4, 8, device=dev)
    with pytest.raises(ValueError, match="rank"):
        ops.quantize_affine(x, [1, 4, 1], torch.ones(8, device=dev), None, "qint8", 0, 0)
    with pytest.raises(ValueError, match="positive"):
        ops.quantize_affine(x, [1, 0], torch.ones(8, device=dev), None, "qint8", 0, 0)
    with pytest.raises(ValueError, match="one entry per block"):
        ops.quantize_affine(x, [1, 4], torch.ones(3, device=dev), None, "qint8", 0, 0)
    with pytest.raises(TypeError):
        ops.quantize_affine(x, [1, 4], torch.ones(8, device=dev), None, torch.float16, 0, 0)
    with pytest.raises(RuntimeError, match="input device"):
        ops.quantize_affine(x, [1, 4], torch.ones(8), None, "qint8", 0, 0)
    with pytest.raises(TypeError):
        ops.dequantize_affine(torch.zeros(4, 8, device=dev), [1, 4], torch.ones(8, device=dev))
    empty = ops.quantize_affine(torch.zeros(0, 8, device=dev), [1, 4], torch.ones(0, device=dev), None, "quint8", 0, 0)
    assert empty.shape == (0, 8) and empty.dtype == torch.uint8
