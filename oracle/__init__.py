"""ctypes front-end of the CPU oracle (``oracle/tpq_oracle.c``).

TEST INFRASTRUCTURE ONLY.  The product package never imports this module; it
is loaded by ``tests/``, by the smoke check and by the benchmark's
``cpu_baseline`` leg, always as the checker and never as the thing measured
or shipped.

All functions take and return numpy arrays.  16-bit float tensors travel as
``uint16`` bit patterns together with a dtype tag (``"f16"`` / ``"bf16"``),
because numpy has no bfloat16.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

F32, F16, BF16 = 0, 1, 2
_DT = {"f32": F32, "f16": F16, "bf16": BF16, F32: F32, F16: F16, BF16: BF16}


def build(force: bool = False) -> str:
    """Compile ``liboracle.so`` with the committed Makefile."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _LIB_PATH


def build_native(directory: str) -> ctypes.CDLL:
    """The same source compiled with ``-march=native`` into `directory`, loaded and returned: the benchmark's CPU
    baseline is timed with the host's full ISA (the library that travels with the repository is built for AVX2 so that
    it runs on any host).  Raises if the compiler is missing or fails."""
    out = os.path.join(directory, "liboracle_native.so")
    flags = ["-O3", "-fPIC", "-std=c11", "-ffp-contract=off", "-fno-fast-math", "-fno-math-errno", "-fvisibility=hidden",
             "-march=native"]
    subprocess.run([os.environ.get("CC", "gcc"), *flags, "-shared", "-o", out, os.path.join(_HERE, "tpq_oracle.c"), "-lm"],
                   check=True, capture_output=True)
    return ctypes.CDLL(out)


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype=None):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def storage(dtype) -> np.dtype:
    return np.dtype(np.float32) if _DT[dtype] == F32 else np.dtype(np.uint16)


def convert(src: np.ndarray, src_dtype, dst_dtype) -> np.ndarray:
    """Convert between f32 / f16-bits / bf16-bits (round to nearest even)."""
    src = _c(src, storage(src_dtype))
    dst = np.empty(src.shape, storage(dst_dtype))
    lib().orc_convert(_p(src), _DT[src_dtype], _p(dst), _DT[dst_dtype], ctypes.c_int64(src.size))
    return dst


def to_f32(a: np.ndarray, dtype) -> np.ndarray:
    return convert(a, dtype, "f32")


def from_f32(a: np.ndarray, dtype) -> np.ndarray:
    return convert(np.asarray(a, np.float32), "f32", dtype)


def quantize_rowwise(x, dtype="f32", eps=1e-5, divisor=127.0, qmin=-127, qmax=127, sign_mode=False):
    x = _c(x, storage(dtype))
    M, K = x.shape
    codes = np.empty((M, K), np.int8)
    scales = np.empty((M,), np.float32)
    lib().orc_quantize_rowwise(_p(x), _DT[dtype], ctypes.c_int64(M), ctypes.c_int64(K),
                               ctypes.c_float(eps), ctypes.c_float(divisor), int(qmin), int(qmax),
                               int(bool(sign_mode)), _p(codes), _p(scales))
    return codes, scales


def quantize_int8_rowwise(x, dtype="f32", eps=1e-5):
    return quantize_rowwise(x, dtype, eps, 127.0, -127, 127, False)


def quantize_int4_rowwise(x, dtype="f32", eps=1e-8):
    return quantize_rowwise(x, dtype, eps, 7.0, -8, 7, False)


def quantize_int2_rowwise(x, dtype="f32", eps=1e-8):
    return quantize_rowwise(x, dtype, eps, 2.0, -2, 1, False)


def quantize_binary_rowwise(x, dtype="f32", eps=1e-8):
    return quantize_rowwise(x, dtype, eps, 1.0, -1, 1, True)


def int_mm(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """C = A @ B with A [M,K] int8/uint8 and B [K,N] int8 (any strides)."""
    a = np.ascontiguousarray(a)
    assert a.dtype in (np.int8, np.uint8) and b.dtype == np.int8
    M, K = a.shape
    K2, N = b.shape
    assert K == K2
    if b.strides == (1, K) and N > 1:
        base, sk, sn = b.T, 1, K
    else:
        b = np.ascontiguousarray(b)
        base, sk, sn = b, N, 1
    c = np.empty((M, N), np.int32)
    lib().orc_int_mm(_p(a), int(a.dtype == np.uint8), _p(base), ctypes.c_int64(sk),
                     ctypes.c_int64(sn), _p(c), ctypes.c_int64(M), ctypes.c_int64(K),
                     ctypes.c_int64(N))
    return c


def int_mm_nk(a: np.ndarray, w: np.ndarray, rows=None) -> np.ndarray:
    a, w = _c(a, np.int8), _c(w, np.int8)
    M, K = a.shape
    N = w.shape[0]
    r0, r1 = (0, M) if rows is None else rows
    c = np.zeros((M, N), np.int32)
    lib().orc_int_mm_nk(_p(a), _p(w), _p(c), ctypes.c_int64(M), ctypes.c_int64(K),
                        ctypes.c_int64(N), ctypes.c_int64(r0), ctypes.c_int64(r1))
    return c


def int8_mm_rescale(acc, rs, cs, bias=None, out_dtype="f32"):
    acc = _c(acc, np.int32)
    M, N = acc.shape
    rs = _c(np.asarray(rs).reshape(-1), np.float32)
    cs = _c(np.asarray(cs).reshape(-1), np.float32)
    bias = None if bias is None else _c(bias, np.float32)
    out = np.empty((M, N), storage(out_dtype))
    lib().orc_int8_mm_rescale(_p(acc), _p(rs), _p(cs), _p(bias), _p(out), _DT[out_dtype],
                              ctypes.c_int64(M), ctypes.c_int64(N))
    return out


def int4_pack_cpu(codes, columns=64, half_split=True):
    codes = _c(codes, np.int32)
    N, K = codes.shape
    out = np.empty((N, K // 2), np.uint8)
    lib().orc_int4_pack_cpu(_p(codes), _p(out), ctypes.c_int64(N), ctypes.c_int64(K), int(columns),
                            int(bool(half_split)))
    return out


def int4_mm_cpu(x, dtype, packed, params, group, columns=64, half_split=True, rows=None):
    x = _c(x, storage(dtype))
    packed = _c(packed, np.uint8)
    params = _c(params, storage(dtype))
    m, k = x.shape
    n = packed.shape[0]
    r0, r1 = (0, m) if rows is None else rows
    out = np.zeros((m, n), storage(dtype))
    lib().orc_int4_mm_cpu(_p(x), _DT[dtype], _p(packed), _p(params), _p(out), ctypes.c_int64(m),
                          ctypes.c_int64(n), ctypes.c_int64(k), ctypes.c_int64(group), int(columns),
                          int(bool(half_split)), ctypes.c_int64(r0), ctypes.c_int64(r1))
    return out


def int4_mm_cpu_blocked(x, dtype, packed, params, group, blocks=None, out=None, library=None):
    """Vectorisable twin of int4_mm_cpu (64-column AVX-512 layout); `blocks` = (begin, end)
    column blocks to compute, so that threads can split the work; `library`: a build_native() library."""
    x = _c(x, storage(dtype))
    packed = _c(packed, np.uint8)
    params = _c(params, storage(dtype))
    m, k = x.shape
    n = packed.shape[0]
    assert n % 64 == 0
    b0, b1 = (0, n // 64) if blocks is None else blocks
    if out is None:
        out = np.zeros((m, n), storage(dtype))
    (library or lib()).orc_int4_mm_cpu_blocked(_p(x), _DT[dtype], _p(packed), _p(params), _p(out), ctypes.c_int64(m),
                                  ctypes.c_int64(n), ctypes.c_int64(k), ctypes.c_int64(group),
                                  ctypes.c_int64(b0), ctypes.c_int64(b1))
    return out


def int4_pack_tc(codes, inner_k_tiles=2):
    codes = _c(codes, np.int32)
    N, K = codes.shape
    n_tiles = (N + 7) // 8
    k_super = (K + inner_k_tiles * 16 - 1) // (inner_k_tiles * 16)
    out = np.empty((n_tiles, k_super, 32, inner_k_tiles // 2), np.int32)
    lib().orc_int4_pack_tc(_p(codes), ctypes.c_int64(N), ctypes.c_int64(K), int(inner_k_tiles),
                           _p(out))
    return out


def int4_unpack_tc(packed, K):
    """Codes [8*nTiles, K] read back through the dequantize kernel's index map."""
    packed = _c(packed, np.int32)
    assert packed.ndim == 4 and packed.shape[2] == 32 and packed.shape[3] == 1
    N = packed.shape[0] * 8
    codes = np.zeros((N, K), np.int32)
    lib().orc_int4_tc_dequantize(_p(packed), None, F32, None, _p(codes), ctypes.c_int64(N),
                                 ctypes.c_int64(K), ctypes.c_int64(32))
    return codes


def int4_dequantize_tc(packed, sz, dtype, K, group):
    packed = _c(packed, np.int32)
    N = packed.shape[0] * 8
    sz = _c(sz, storage(dtype))
    W = np.zeros((N, K), storage(dtype))
    lib().orc_int4_tc_dequantize(_p(packed), _p(sz), _DT[dtype], _p(W), None, ctypes.c_int64(N),
                                 ctypes.c_int64(K), ctypes.c_int64(group))
    return W


def int4_mm_tc(x, dtype, packed, sz, group, round_w=True, want_f64=False, rows=None):
    x = _c(x, storage(dtype))
    packed = _c(packed, np.int32)
    sz = _c(sz, storage(dtype))
    M, K = x.shape
    N = packed.shape[0] * 8
    r0, r1 = (0, M) if rows is None else rows
    out = np.zeros((M, N), storage(dtype))
    y64 = np.zeros((M, N), np.float64) if want_f64 else None
    lib().orc_int4_mm_tc(_p(x), _DT[dtype], _p(packed), _p(sz), _p(out), _p(y64), ctypes.c_int64(M),
                         ctypes.c_int64(N), ctypes.c_int64(K), ctypes.c_int64(group),
                         int(bool(round_w)), ctypes.c_int64(r0), ctypes.c_int64(r1))
    return (out, y64) if want_f64 else out


def pack_ternary(codes):
    codes = _c(codes, np.int8)
    lead, cols = codes.shape[:-1], codes.shape[-1]
    flat = codes.reshape(-1, cols)
    out = np.empty((flat.shape[0], (cols + 3) // 4), np.uint8)
    lib().orc_pack_ternary(_p(flat), ctypes.c_int64(flat.shape[0]), ctypes.c_int64(cols), _p(out))
    return out.reshape(*lead, (cols + 3) // 4)


def unpack_ternary(packed, columns):
    packed = _c(packed, np.uint8)
    lead = packed.shape[:-1]
    flat = packed.reshape(-1, packed.shape[-1])
    cols = min(columns, flat.shape[1] * 4)
    out = np.empty((flat.shape[0], cols), np.int8)
    lib().orc_unpack_ternary(_p(flat), ctypes.c_int64(flat.shape[0]), ctypes.c_int64(cols), _p(out))
    return out.reshape(*lead, cols)


def bitnet_scale(w, eps=1e-5) -> np.float32:
    """mean(|W|) clamped to eps (bitnet.py:48-54); summed in double, returned as fp32."""
    return np.float32(max(float(np.abs(np.asarray(w, np.float64)).mean()), eps))


def quantize_bitnet_weight(w, scale=None, eps=1e-5):
    w = _c(w, np.float32)
    scale = bitnet_scale(w, eps) if scale is None else np.float32(max(float(scale), eps))
    codes = np.empty(w.shape, np.int8)
    lib().orc_quantize_bitnet_weight(_p(w), ctypes.c_int64(w.size), ctypes.c_float(scale), _p(codes))
    return codes, scale


def weight_prepack(w):
    w = _c(w, np.int8)
    N, K = w.shape
    packed = np.empty((N, (K + 31) // 32 * 32), np.int8)
    offsets = np.empty((N,), np.int64)
    lib().orc_weight_prepack(_p(w), ctypes.c_int64(N), ctypes.c_int64(K), _p(packed), _p(offsets))
    return packed, offsets


def packed_run_linear_float(x, xs, xz, packed, offsets, ws, wz, bias, K):
    x = np.ascontiguousarray(x)
    rows = x.shape[0]
    N = packed.shape[0]
    ws, wz = _c(ws, np.float32), _c(wz, np.int64)
    bias = None if bias is None else _c(bias, np.float32)
    out = np.empty((rows, N), np.float32)
    lib().orc_packed_run_linear_float(_p(x), int(x.dtype == np.uint8), ctypes.c_double(xs),
                                      ctypes.c_int64(xz), _p(_c(packed, np.int8)),
                                      _p(_c(offsets, np.int64)), _p(ws), _p(wz), _p(bias), _p(out),
                                      ctypes.c_int64(rows), ctypes.c_int64(N), ctypes.c_int64(K))
    return out


def ternary_mm(x_i8, row_scale, packed, w_scale, K, bias=None, out_dtype="f32"):
    x_i8 = _c(x_i8, np.int8)
    packed = _c(packed, np.uint8)
    M = x_i8.shape[0]
    N = packed.shape[0]
    rs = _c(np.asarray(row_scale).reshape(-1), np.float32)
    bias = None if bias is None else _c(bias, np.float32)
    out = np.empty((M, N), storage(out_dtype))
    acc = np.empty((M, N), np.int32)
    lib().orc_ternary_mm(_p(x_i8), _p(rs), _p(packed), ctypes.c_float(w_scale), _p(bias),
                         ctypes.c_int64(M), ctypes.c_int64(N), ctypes.c_int64(K), _p(out),
                         _DT[out_dtype], _p(acc))
    return out, acc


def weight_int8pack_mm(x, dtype, w, scales, want_f64=False):
    x = _c(x, storage(dtype))
    w = _c(w, np.int8)
    scales = _c(scales, np.float32)
    M, K = x.shape
    N = w.shape[0]
    out = np.zeros((M, N), storage(dtype))
    y64 = np.zeros((M, N), np.float64) if want_f64 else None
    lib().orc_weight_int8pack_mm(_p(x), _DT[dtype], _p(w), _p(scales), ctypes.c_int64(M), ctypes.c_int64(N),
                                 ctypes.c_int64(K), _p(out), _p(y64))
    return (out, y64) if want_f64 else out


def rms_norm(x, dtype, weight=None, eps=1e-5, want_f64=False):
    """rms_norm over the last dimension of a 2-D array of storage bits / float32; weight: [K] of the same type or None."""
    x = _c(x, storage(dtype))
    M, K = x.shape
    weight = None if weight is None else _c(weight, storage(dtype))
    out = np.zeros((M, K), storage(dtype))
    y64 = np.zeros((M, K), np.float64) if want_f64 else None
    lib().orc_rms_norm(_p(x), _DT[dtype], ctypes.c_int64(M), ctypes.c_int64(K), _p(weight), ctypes.c_float(eps), _p(out), _p(y64))
    return (out, y64) if want_f64 else out


AFFINE_STORAGE = {"qint8": (0, np.int8, 1), "quint8": (1, np.uint8, 1), "qint32": (2, np.int32, 1),
                  "quint4x2": (3, np.uint8, 2), "quint2x4": (4, np.uint8, 4), "quint1x8": (5, np.uint8, 8)}
_AFFINE_BOUNDS = {"qint8": (-128, 127), "quint8": (0, 255), "qint32": (-2**31, 2**31 - 1),
                  "quint4x2": (0, 15), "quint2x4": (0, 3), "quint1x8": (0, 1)}


def _affine_common(shape, block_size, scales, zeros):
    arr = ctypes.c_int64 * max(len(shape), 1)
    scales = _c(np.asarray(scales, np.float32).reshape(-1), np.float32)
    zeros = None if zeros is None else _c(np.asarray(zeros, np.float32).reshape(-1), np.float32)
    return arr(*shape), arr(*block_size), scales, zeros


def quantize_affine(x, block_size, scales, zeros, dtype, quant_min=0, quant_max=0):
    """Codes of `dtype` ("qint8" ... "quint1x8"): an array of x's shape, or the flat packed bytes."""
    x = _c(x, np.float32)
    tag, code_dtype, pack = AFFINE_STORAGE[dtype]
    lo, hi = _AFFINE_BOUNDS[dtype]
    qmin = quant_min if quant_min < quant_max else lo   # QuantKernels.cpp:619-622
    qmax = quant_max if quant_max > quant_min else hi
    sizes, blocks, scales, zeros = _affine_common(x.shape, block_size, scales, zeros)
    out = np.zeros(x.shape, code_dtype) if pack == 1 else np.zeros(((x.size + pack - 1) // pack,), np.uint8)
    lib().orc_quantize_affine(_p(x), ctypes.c_int(x.ndim), sizes, blocks, _p(scales), ctypes.c_int64(scales.size),
                              _p(zeros), ctypes.c_int64(0 if zeros is None else zeros.size), ctypes.c_int(tag),
                              ctypes.c_int64(qmin), ctypes.c_int64(qmax), _p(out))
    return out


def dequantize_affine(codes, shape, block_size, scales, zeros, dtype):
    tag, code_dtype, _ = AFFINE_STORAGE[dtype]
    codes = _c(codes, code_dtype)
    sizes, blocks, scales, zeros = _affine_common(tuple(shape), block_size, scales, zeros)
    out = np.zeros(tuple(shape), np.float32)
    lib().orc_dequantize_affine(_p(codes), ctypes.c_int(tag), ctypes.c_int(len(shape)), sizes, blocks, _p(scales),
                                ctypes.c_int64(scales.size), _p(zeros), ctypes.c_int64(0 if zeros is None else zeros.size),
                                _p(out))
    return out


def lowbit_pack(codes, bits, lsb_first=False):
    codes = _c(codes, np.uint8)
    rows, cols = codes.shape
    per_byte = 8 // bits
    out = np.zeros((rows, (cols + per_byte - 1) // per_byte), np.uint8)
    lib().orc_lowbit_pack(_p(codes), ctypes.c_int(bits), ctypes.c_int(int(lsb_first)), ctypes.c_int64(rows), ctypes.c_int64(cols), _p(out))
    return out


def lowbit_unpack(packed, bits, cols, lsb_first=False):
    packed = _c(packed, np.uint8)
    rows = packed.shape[0]
    out = np.zeros((rows, cols), np.uint8)
    lib().orc_lowbit_unpack(_p(packed), ctypes.c_int(bits), ctypes.c_int(int(lsb_first)), ctypes.c_int64(rows), ctypes.c_int64(cols), _p(out))
    return out


def lowbit_mm(x, dtype, packed, bits, sz, K, group, bias=None, lsb_first=False, want_f64=False, want_dense=False):
    """(out, [y64], [dense]) of the packed n-bit weight-only linear; sz is float32 [K // group, N, 2]."""
    packed = _c(packed, np.uint8)
    sz = _c(sz, np.float32)
    N = packed.shape[0]
    x = None if x is None else _c(x, storage(dtype))
    M = 0 if x is None else x.shape[0]
    bias = None if bias is None else _c(bias, np.float32)
    out = np.zeros((M, N), storage(dtype))
    y64 = np.zeros((M, N), np.float64) if want_f64 else None
    dense = np.zeros((N, K), np.float32) if want_dense else None
    lib().orc_lowbit_mm(_p(x), _DT[dtype], _p(packed), ctypes.c_int(bits), ctypes.c_int(int(lsb_first)), _p(sz), _p(bias),
                        ctypes.c_int64(M), ctypes.c_int64(N), ctypes.c_int64(K), ctypes.c_int64(group), _p(out), _p(y64), _p(dense))
    res = (out,) + ((y64,) if want_f64 else ()) + ((dense,) if want_dense else ())
    return res if len(res) > 1 else out
