#!/usr/bin/env python3
"""Writes tests/golden/quant_path_vectors.npz: small input/expected-output vectors for the
quantized-linear path.

Inputs are regenerated from the seeded numpy generators the reference's own tests use
(default_rng(124) int4, test/quantization/test_native_operator_families.py:583-590;
default_rng(23) packed linear, test_packed_quantization.py:44-46; the BitNet literals of
test_native_1bit.py:215-216 and :228-229).  Expected outputs come from routines that are
independent of this repository's oracle: PyTorch CPU library ops where the reference asserts
equality with them (`_convert_weight_to_int4pack_for_cpu`, `_weight_int4pack_mm_for_cpu`,
`_int_mm`), and the closed forms written out in the reference tests (numpy, int64 / float32).

Run:  python tests/golden/make_fixtures.py
"""
import os

import numpy as np
import torch

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "quant_path_vectors.npz")
v = {}

# ---- int4: CPU layout and multiply (library pin), codes reused for the device layout -------------
for tag, channels, group, rows in (("a", 64, 32, 5), ("b", 48, 64, 1), ("c", 128, 128, 33)):
    rng = np.random.default_rng(124)
    features = group * 2
    codes = rng.integers(0, 16, size=(channels, features), dtype="int32")
    data = rng.normal(0, .2, size=(rows, features)).astype("float32")
    params = rng.uniform(-.05, .05, size=(2, channels, 2)).astype("float32")
    packed = torch._convert_weight_to_int4pack_for_cpu(torch.tensor(codes), 2)
    v[f"int4_{tag}_codes"] = codes
    v[f"int4_{tag}_x"] = data
    v[f"int4_{tag}_params"] = params
    v[f"int4_{tag}_group"] = np.int64(group)
    v[f"int4_{tag}_packed_cpu"] = packed.numpy()
    for dt, tdt in (("f32", torch.float32), ("f16", torch.float16), ("bf16", torch.bfloat16)):
        y = torch._weight_int4pack_mm_for_cpu(torch.tensor(data).to(tdt), packed, group, torch.tensor(params).to(tdt))
        v[f"int4_{tag}_y_{dt}"] = y.float().numpy()
    # fp64 truth of the same quantized weights: y = x . ((code - 8) s + z)
    s = np.repeat(params[:, :, 0].T.astype(np.float64), group, axis=1)
    z = np.repeat(params[:, :, 1].T.astype(np.float64), group, axis=1)
    v[f"int4_{tag}_y_f64"] = data.astype(np.float64) @ ((codes - 8) * s + z).T

# ---- int8: rowwise quantizer closed form, integer product, rescale ------------------------------
rng = np.random.default_rng(7)
x = rng.normal(0, 1, (16, 256)).astype(np.float32)
w = rng.normal(0, 0.02, (192, 256)).astype(np.float32)
bias = rng.normal(0, 0.01, (192,)).astype(np.float32)


def rowwise(a):
    absmax = np.maximum(np.abs(a).max(axis=-1, keepdims=True), np.float32(1e-5)).astype(np.float32)
    scale = (absmax / np.float32(127.0)).astype(np.float32)
    codes = np.clip(np.rint((a / scale).astype(np.float32)), -127, 127).astype(np.int8)
    return codes, scale[:, 0]


xq, xs = rowwise(x)
wq, ws = rowwise(w)
acc = torch._int_mm(torch.from_numpy(np.vstack([xq, xq])), torch.from_numpy(wq).t()).numpy()[:16]  # torch wants M > 16
assert np.array_equal(acc, xq.astype(np.int64) @ wq.astype(np.int64).T)
res = (acc.astype(np.float32) * xs[:, None]) * ws[None, :]
v.update(int8_x=x, int8_w=w, int8_bias=bias, int8_xq=xq, int8_xs=xs, int8_wq=wq, int8_ws=ws, int8_acc=acc,
         int8_rescaled=res.astype(np.float32), int8_linear=(res + bias[None, :]).astype(np.float32))

# ---- BitNet literals and closed forms ---------------------------------------------------------------
wlit = np.array([[.4, -.1, .2, -.3], [.0, .6, -.8, .1]], np.float32)
scale = np.abs(wlit).mean(dtype=np.float32)
v["bitnet_lit_w"] = wlit
v["bitnet_lit_scale"] = np.float32(scale)
v["bitnet_lit_codes"] = np.clip(np.round(wlit / scale), -1, 1).astype(np.int8)
tern = np.array([[1, -1, 0, 1, -1, 0, 0, 1, -1], [0, 1, -1, -1, 1, 0, 1, -1, 0]], np.int8)
pad = np.concatenate([tern, np.zeros((2, 3), np.int8)], axis=1).astype(np.int32)
v["ternary_lit_codes"] = tern
v["ternary_lit_packed"] = (((pad[:, 0::4] & 3) << 6) | ((pad[:, 1::4] & 3) << 4) | ((pad[:, 2::4] & 3) << 2) | (pad[:, 3::4] & 3)).astype(np.uint8)
rng = np.random.default_rng(611)
bw = rng.normal(0, 0.05, (24, 36)).astype(np.float32)
bx = rng.normal(0, 1, (5, 36)).astype(np.float32)
bscale = np.abs(bw).mean(dtype=np.float32)
bcodes = np.clip(np.round(bw / bscale), -1, 1).astype(np.int32)
bxq, bxs = rowwise(bx)
v.update(bitnet_w=bw, bitnet_x=bx, bitnet_scale=np.float32(bscale), bitnet_codes=bcodes.astype(np.int8),
         bitnet_y=((bxq.astype(np.int32) @ bcodes.T).astype(np.float32) * bxs[:, None] * bscale).astype(np.float32))

# ---- packed int8 linear, integer closed form (xs=1, xz=0, ws=1, wz=0 is the hot-path case) ---------
for K in (3, 31, 32, 65):
    rng = np.random.default_rng(23)
    xcodes = rng.integers(-128, 128, (2, 3, K), dtype=np.int16)
    wcodes = rng.integers(-128, 128, (7, K), dtype=np.int16)
    v[f"packed_K{K}_x"] = xcodes.astype(np.int8)
    v[f"packed_K{K}_w"] = wcodes.astype(np.int8)
    v[f"packed_K{K}_offsets"] = wcodes.astype(np.int64).sum(1)
    v[f"packed_K{K}_acc"] = (xcodes.astype(np.int64) @ wcodes.astype(np.int64).T).astype(np.int32)

# ---- int8 weight-only matmul: the literal example of test/test_mps.py:1052-1061 and a seeded case --
a_lit = np.array([[0.5, -1.0, 2.0, 0.25], [1.0, 0.5, -0.5, 2.0]], np.float32)
w_lit = np.array([[1, -2, 0, 1], [0, 1, -1, 2], [2, 0, 1, -1]], np.int8)
s_lit = np.array([0.5, 1.0, 2.0], np.float32)
v.update(int8pack_lit_a=a_lit, int8pack_lit_w=w_lit, int8pack_lit_s=s_lit,
         int8pack_lit_y=((a_lit @ w_lit.astype(np.float32).T) * s_lit).astype(np.float32))
rng = np.random.default_rng(901)
pa = rng.normal(0, 1, (3, 256)).astype(np.float32)
pw = rng.integers(-128, 128, (40, 256)).astype(np.int8)
ps = rng.uniform(0.001, 0.02, 40).astype(np.float32)
v.update(int8pack_a=pa, int8pack_w=pw, int8pack_s=ps,
         int8pack_y_f64=(pa.astype(np.float64) @ pw.astype(np.float64).T) * ps.astype(np.float64))

# ---- quantize_affine: PyTorch CPU twins (one block, per-row blocks) and the grouped closed form -----
rng = np.random.default_rng(902)
qa = (rng.standard_normal((6, 40)) * 30).astype(np.float32)
qa[0, :8] = np.array([-.5, .5, 1.5, 2.5, 3.5, 4.5, 7.5, 15.5], np.float32) * np.float32(0.37)  # ties
v["affine_x"] = qa
v["affine_tensor_scale"], v["affine_tensor_zero"] = np.float32(0.37), np.float32(3)
for name, tdt in (("qint8", torch.qint8), ("quint8", torch.quint8)):
    q = torch.quantize_per_tensor(torch.from_numpy(qa), 0.37, 3, tdt)
    v[f"affine_tensor_{name}"] = q.int_repr().numpy()
    v[f"affine_tensor_{name}_back"] = q.dequantize().numpy()
row_s = rng.uniform(0.05, 0.9, 6).astype(np.float32)
row_z = rng.integers(-4, 5, 6).astype(np.float32)
q = torch.quantize_per_channel(torch.from_numpy(qa), torch.from_numpy(row_s).double(), torch.from_numpy(row_z).long(), 0, torch.qint8)
v.update(affine_row_scale=row_s, affine_row_zero=row_z, affine_row_qint8=q.int_repr().numpy(), affine_row_back=q.dequantize().numpy())
grp_s = rng.uniform(0.5, 4.0, (6, 5)).astype(np.float32)   # groups of 8 along the rows
grp_z = np.full((6, 5), 8.0, np.float32)
inv = (np.float32(1) / grp_s).astype(np.float32)
pos = np.rint((qa.reshape(6, 5, 8) * inv[:, :, None]).astype(np.float32)) + grp_z[:, :, None]
codes4 = np.clip(pos, 0, 15).astype(np.uint8).reshape(6, 40)
v.update(affine_group_scale=grp_s, affine_group_zero=grp_z, affine_group_u4_codes=codes4,
         affine_group_u4_packed=(codes4.reshape(-1)[0::2] | (codes4.reshape(-1)[1::2] << 4)).astype(np.uint8),  # low bits first
         affine_group_u4_back=((codes4.reshape(6, 5, 8).astype(np.float32) - grp_z[:, :, None]) * grp_s[:, :, None]).reshape(6, 40).astype(np.float32))

# ---- packed n-bit weight-only linear: the reference's pack formulas and x @ dq.T --------------------
rng = np.random.default_rng(903)
for bits in (1, 2, 4):
    per_byte = 8 // bits
    lc = rng.integers(0, 1 << bits, (12, 40)).astype(np.int32)
    packed = np.zeros((12, 40 // per_byte), np.int32)
    for i in range(per_byte):  # pack_intx: code i of a byte at shift 8 - (i + 1) * bits
        packed |= (lc[:, i::per_byte] & ((1 << bits) - 1)) << (8 - (i + 1) * bits)
    lsz = np.stack([rng.uniform(0.01, 0.2, (5, 12)), rng.integers(0, 1 << bits, (5, 12)).astype(np.float64)], axis=-1).astype(np.float32)
    dq = ((lc.astype(np.float32) - np.repeat(lsz[:, :, 1].T, 8, axis=1)) * np.repeat(lsz[:, :, 0].T, 8, axis=1)).astype(np.float32)
    lx = rng.standard_normal((3, 40)).astype(np.float32)
    v.update({f"lowbit{bits}_codes": lc.astype(np.uint8), f"lowbit{bits}_packed": packed.astype(np.uint8), f"lowbit{bits}_sz": lsz,
              f"lowbit{bits}_x": lx, f"lowbit{bits}_dense": dq, f"lowbit{bits}_y_f64": lx.astype(np.float64) @ dq.astype(np.float64).T})
sign = rng.integers(0, 2, (4, 10)).astype(np.uint8)       # pack_binary: code i of a byte in bit i, zero padded
padded = np.zeros((4, 16), np.uint8); padded[:, :10] = sign
v.update(binary_codes=sign, binary_packed=sum(((padded[:, i::8] & 1) << i) for i in range(8)).astype(np.uint8))

np.savez_compressed(OUT, **v)
print(OUT, os.path.getsize(OUT), "bytes,", len(v), "arrays")
