"""The committed golden vectors (tests/golden/quant_path_vectors.npz, written by
tests/golden/make_fixtures.py from PyTorch CPU library ops and the reference tests' closed forms)
against the CPU oracle (not gpu) and against the HIP library (gpu)."""
import os

import numpy as np
import pytest

import oracle
from helpers import cast_bits, from_bits

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "quant_path_vectors.npz"))
INT4_TOL = {"f32": (2e-5, 2e-5), "f16": (2e-4, 2e-3), "bf16": (2e-3, 2e-2)}  # the reference test's atol, rtol


@pytest.mark.parametrize("tag", ["a", "b", "c"])
def test_oracle_int4_cpu_layout_and_mm(tag):
    codes, group = G[f"int4_{tag}_codes"], int(G[f"int4_{tag}_group"])
    packed = oracle.int4_pack_cpu(codes, 64, True)
    np.testing.assert_array_equal(packed, G[f"int4_{tag}_packed_cpu"])
    for dt in ("f32", "f16", "bf16"):
        got = oracle.int4_mm_cpu(cast_bits(G[f"int4_{tag}_x"], dt), dt, packed, cast_bits(G[f"int4_{tag}_params"], dt), group)
        np.testing.assert_array_equal(oracle.to_f32(got, dt), G[f"int4_{tag}_y_{dt}"])  # bit-exact with torch CPU


@pytest.mark.parametrize("tag", ["a", "b", "c"])
def test_oracle_int4_device_layout_mm_close_to_f64(tag):
    codes, group = G[f"int4_{tag}_codes"], int(G[f"int4_{tag}_group"])
    packed = oracle.int4_pack_tc(codes, 2)
    np.testing.assert_array_equal(oracle.int4_unpack_tc(packed, codes.shape[1])[: codes.shape[0]], codes)
    for dt in ("f32", "f16", "bf16"):
        got = oracle.int4_mm_tc(cast_bits(G[f"int4_{tag}_x"], dt), dt, packed, cast_bits(G[f"int4_{tag}_params"], dt), group)
        atol, rtol = INT4_TOL[dt]
        np.testing.assert_allclose(oracle.to_f32(got, dt)[:, : codes.shape[0]], G[f"int4_{tag}_y_{dt}"], atol=5 * atol, rtol=5 * rtol)


def test_oracle_int8_chain():
    xq, xs = oracle.quantize_int8_rowwise(G["int8_x"], "f32", 1e-5)
    wq, ws = oracle.quantize_int8_rowwise(G["int8_w"], "f32", 1e-5)
    np.testing.assert_array_equal(xq, G["int8_xq"]); np.testing.assert_array_equal(xs, G["int8_xs"])
    np.testing.assert_array_equal(wq, G["int8_wq"]); np.testing.assert_array_equal(ws, G["int8_ws"])
    acc = oracle.int_mm_nk(xq, wq)
    np.testing.assert_array_equal(acc, G["int8_acc"])
    np.testing.assert_array_equal(oracle.int8_mm_rescale(acc, xs, ws), G["int8_rescaled"])
    np.testing.assert_array_equal(oracle.int8_mm_rescale(acc, xs, ws, bias=G["int8_bias"]), G["int8_linear"])


def test_oracle_bitnet():
    np.testing.assert_array_equal(oracle.bitnet_scale(G["bitnet_lit_w"]), G["bitnet_lit_scale"])
    codes, _ = oracle.quantize_bitnet_weight(G["bitnet_lit_w"])
    np.testing.assert_array_equal(codes, G["bitnet_lit_codes"])
    np.testing.assert_array_equal(oracle.pack_ternary(G["ternary_lit_codes"]), G["ternary_lit_packed"])
    np.testing.assert_array_equal(oracle.unpack_ternary(G["ternary_lit_packed"], 9), G["ternary_lit_codes"])
    codes, scale = oracle.quantize_bitnet_weight(G["bitnet_w"])
    np.testing.assert_array_equal(codes, G["bitnet_codes"])
    xq, xs = oracle.quantize_int8_rowwise(G["bitnet_x"], "f32", 1e-5)
    y, _ = oracle.ternary_mm(xq, xs, oracle.pack_ternary(codes), float(scale), 36)
    np.testing.assert_allclose(y, G["bitnet_y"], rtol=1e-5, atol=1e-5)  # the reference test's tolerance


@pytest.mark.parametrize("K", [3, 31, 32, 65])
def test_oracle_packed_linear(K):
    x, w = G[f"packed_K{K}_x"].reshape(-1, K), G[f"packed_K{K}_w"]
    packed, offsets = oracle.weight_prepack(w)
    assert packed.shape == (7, ((K + 31) // 32) * 32)
    np.testing.assert_array_equal(offsets, G[f"packed_K{K}_offsets"])
    y = oracle.packed_run_linear_float(x, 1.0, 0, packed, offsets, np.ones(7, np.float32), np.zeros(7, np.int64), None, K)
    np.testing.assert_array_equal(y, G[f"packed_K{K}_acc"].reshape(-1, 7).astype(np.float32))


# ---- the same vectors through the HIP library -------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["a", "b", "c"])
def test_gpu_int4_device_path(tag):
    import torch
    from gpu_util import dev, host
    from tensorplay_amd import ops

    codes, group = G[f"int4_{tag}_codes"], int(G[f"int4_{tag}_group"])
    packed = ops._convert_weight_to_int4pack(dev(codes), 2)
    np.testing.assert_array_equal(host(packed), oracle.int4_pack_tc(codes, 2))
    for dt in ("f32", "f16", "bf16"):
        x = dev(cast_bits(G[f"int4_{tag}_x"], dt), dt)
        sz = dev(cast_bits(G[f"int4_{tag}_params"], dt), dt)
        y = ops._weight_int4pack_mm(x, packed, group, sz).float().cpu().numpy()
        atol, rtol = INT4_TOL[dt]
        np.testing.assert_allclose(y, G[f"int4_{tag}_y_{dt}"], atol=5 * atol, rtol=5 * rtol)
        want = G[f"int4_{tag}_y_f64"]
        assert np.abs(y - want).max() <= 1e-2 * np.abs(want).max()  # stated tolerance for 16-bit outputs


@pytest.mark.gpu
def test_gpu_int8_chain():
    from gpu_util import dev, host
    from tensorplay_amd import ops

    xq, xs = ops._quantize_int8_rowwise(dev(G["int8_x"]), 1e-5)
    wq, ws = ops._quantize_int8_rowwise(dev(G["int8_w"]), 1e-5)
    np.testing.assert_array_equal(host(xq), G["int8_xq"]); np.testing.assert_array_equal(host(xs), G["int8_xs"])
    np.testing.assert_array_equal(host(wq), G["int8_wq"]); np.testing.assert_array_equal(host(ws), G["int8_ws"])
    acc = ops._int_mm(xq, wq.t())
    np.testing.assert_array_equal(host(acc), G["int8_acc"])
    np.testing.assert_array_equal(host(ops._int8_mm_rescale(acc, xs, ws)), G["int8_rescaled"])
    np.testing.assert_array_equal(host(ops.int8_mm_dequant(xq, wq, xs, ws, dev(G["int8_bias"]))), G["int8_linear"])


@pytest.mark.gpu
def test_gpu_bitnet():
    import torch
    from gpu_util import dev, host
    from tensorplay_amd.ao.quantization import (bitnet_linear_packed, get_bitnet_scale, pack_ternary,
                                                quantize_bitnet_weight, unpack_ternary)

    w = dev(G["bitnet_lit_w"])
    scale = get_bitnet_scale(w)
    np.testing.assert_allclose(scale.item(), G["bitnet_lit_scale"], rtol=1e-6)
    codes, _ = quantize_bitnet_weight(w, scale)
    np.testing.assert_array_equal(host(codes), G["bitnet_lit_codes"])
    packed = pack_ternary(dev(G["ternary_lit_codes"]))
    np.testing.assert_array_equal(host(packed), G["ternary_lit_packed"])
    np.testing.assert_array_equal(host(unpack_ternary(packed, 9)), G["ternary_lit_codes"])
    codes, scale = quantize_bitnet_weight(dev(G["bitnet_w"]))
    np.testing.assert_array_equal(host(codes), G["bitnet_codes"])
    y = bitnet_linear_packed(dev(G["bitnet_x"]), pack_ternary(codes), scale, 36)
    np.testing.assert_allclose(host(y), G["bitnet_y"], rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("K", [3, 31, 32, 65])
def test_gpu_packed_linear_special_case(K):
    """PackedWeight.run with unit scales and zero offsets is float(int dot): the generic _int_mm path."""
    from gpu_util import dev, host
    from tensorplay_amd import ops

    x, w = G[f"packed_K{K}_x"].reshape(-1, K), G[f"packed_K{K}_w"]
    acc = ops._int_mm(dev(x), dev(w).t())
    np.testing.assert_array_equal(host(acc), G[f"packed_K{K}_acc"].reshape(-1, 7))


# ---- the rows next to the path: int8 weight-only, affine quantizer, packed n-bit linears ------------

def test_oracle_int8pack():
    np.testing.assert_allclose(oracle.to_f32(oracle.weight_int8pack_mm(G["int8pack_lit_a"], "f32", G["int8pack_lit_w"], G["int8pack_lit_s"]), "f32"),
                               G["int8pack_lit_y"], atol=1e-5)
    got = oracle.to_f32(oracle.weight_int8pack_mm(G["int8pack_a"], "f32", G["int8pack_w"], G["int8pack_s"]), "f32")
    np.testing.assert_allclose(got, G["int8pack_y_f64"], rtol=1e-5, atol=1e-5)


def _affine_cases():
    x = G["affine_x"]
    yield "qint8", x.shape, [G["affine_tensor_scale"]], [G["affine_tensor_zero"]], G["affine_tensor_qint8"], G["affine_tensor_qint8_back"]
    yield "quint8", x.shape, [G["affine_tensor_scale"]], [G["affine_tensor_zero"]], G["affine_tensor_quint8"], G["affine_tensor_quint8_back"]
    yield "qint8", (1, x.shape[1]), G["affine_row_scale"], G["affine_row_zero"], G["affine_row_qint8"], G["affine_row_back"]
    yield "quint4x2", (1, 8), G["affine_group_scale"], G["affine_group_zero"], G["affine_group_u4_packed"], G["affine_group_u4_back"]


def test_oracle_affine():
    x = G["affine_x"]
    for dtype, block, scales, zeros, want, back in _affine_cases():
        got = oracle.quantize_affine(x, block, scales, zeros, dtype)
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(oracle.dequantize_affine(got, x.shape, block, scales, zeros, dtype), back)


def test_oracle_lowbit():
    for bits in (1, 2, 4):
        np.testing.assert_array_equal(oracle.lowbit_pack(G[f"lowbit{bits}_codes"], bits), G[f"lowbit{bits}_packed"])
        out, y64, dense = oracle.lowbit_mm(G[f"lowbit{bits}_x"], "f32", G[f"lowbit{bits}_packed"], bits, G[f"lowbit{bits}_sz"], 40, 8,
                                           want_f64=True, want_dense=True)
        np.testing.assert_array_equal(dense, G[f"lowbit{bits}_dense"])
        np.testing.assert_allclose(y64, G[f"lowbit{bits}_y_f64"], rtol=1e-12, atol=1e-12)
    np.testing.assert_array_equal(oracle.lowbit_pack(G["binary_codes"], 1, lsb_first=True), G["binary_packed"])


@pytest.mark.gpu
def test_gpu_int8pack():
    from gpu_util import dev, host
    from tensorplay_amd import ops
    np.testing.assert_allclose(host(ops._weight_int8pack_mm(dev(G["int8pack_lit_a"]), dev(G["int8pack_lit_w"]), dev(G["int8pack_lit_s"]))),
                               G["int8pack_lit_y"], atol=1e-5)
    got = host(ops._weight_int8pack_mm(dev(G["int8pack_a"]), dev(G["int8pack_w"]), dev(G["int8pack_s"])))
    np.testing.assert_allclose(got, G["int8pack_y_f64"], rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
def test_gpu_affine():
    from gpu_util import dev, host
    from tensorplay_amd import ops
    x = dev(G["affine_x"])
    for dtype, block, scales, zeros, want, back in _affine_cases():
        sc, zp = dev(np.asarray(scales, np.float32)), dev(np.asarray(zeros, np.float32))
        q = ops.quantize_affine(x, list(block), sc, zp, dtype, 0, 0)
        raw = q.data if isinstance(q, ops.PackedCodes) else q
        np.testing.assert_array_equal(host(raw), want)
        np.testing.assert_array_equal(host(ops.dequantize_affine(q, list(block), sc, zp)), back)


@pytest.mark.gpu
def test_gpu_lowbit():
    from gpu_util import dev, host
    from tensorplay_amd import ops
    for bits in (1, 2, 4):
        packed = ops.pack_lowbit(dev(G[f"lowbit{bits}_codes"]), bits)
        np.testing.assert_array_equal(host(packed), G[f"lowbit{bits}_packed"])
        sz = dev(G[f"lowbit{bits}_sz"])
        np.testing.assert_array_equal(host(ops._lowbit_dequantize(packed, bits, 40, sz)), G[f"lowbit{bits}_dense"])
        np.testing.assert_allclose(host(ops._lowbit_mm(dev(G[f"lowbit{bits}_x"]), packed, bits, 40, sz)), G[f"lowbit{bits}_y_f64"],
                                   rtol=1e-5, atol=1e-5)
    np.testing.assert_array_equal(host(ops.pack_lowbit(dev(G["binary_codes"]), 1, lsb_first=True)), G["binary_packed"])
