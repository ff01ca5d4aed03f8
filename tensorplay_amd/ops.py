"""The quantized-linear native operators, under the names and argument orders the
reference's Python calls them with (``tp._C.<op>`` / ``tp.ops.tp.<op>``), over
PyTorch-ROCm tensors.  Every function validates like the reference's device op,
allocates the result like it, and enqueues the gfx950 kernel on the current
stream through the C ABI of ``include/tpq.h``; none of them synchronises.

Signatures: ``config/native_functions.yaml:5338-5350, 7987-7993`` of the reference.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _lib

_DT = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}
_ERRORS = {
    _lib.TPQ_ERR_INVALID_VALUE: ValueError,
    _lib.TPQ_ERR_INVALID_TYPE: TypeError,
    _lib.TPQ_ERR_RUNTIME: RuntimeError,
    _lib.TPQ_ERR_UNSUPPORTED: NotImplementedError,
}


def _check(status: int) -> None:
    if status != _lib.TPQ_OK:
        raise _ERRORS.get(status, RuntimeError)(_lib.last_error())


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None or t.numel() == 0 else t.data_ptr()


def _require_device(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{what}: expected a tensor on the GPU; this build has no CPU kernels")


def _quantize_rowwise(self, eps, divisor, qmin, qmax, sign_mode, name):
    if self.dim() != 2:
        raise ValueError(f"{name}(): expected a 2-D tensor")
    if self.dtype not in _DT:
        raise TypeError("rowwise quantize: unsupported input dtype")
    _require_device(self, name)
    x = self.contiguous()
    M, K = x.shape
    codes = torch.empty((M, K), dtype=torch.int8, device=x.device)
    scales = torch.empty((M,), dtype=torch.float32, device=x.device)
    if M == 0 or K == 0:
        return codes, scales
    with torch.cuda.device(x.device):
        _check(_lib.load().tpq_quantize_rowwise(_ptr(x), _DT[x.dtype], M, K, float(eps), divisor, qmin,
                                                qmax, int(sign_mode), _ptr(codes), _ptr(scales), _stream(x)))
    return codes, scales


def _quantize_int8_rowwise(self: torch.Tensor, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """codes int8 [M,K] in [-127,127], scales f32 [M] = max(absmax, eps) / 127."""
    return _quantize_rowwise(self, eps, 127.0, -127, 127, False, "_quantize_int8_rowwise")


def _quantize_int4_rowwise(self: torch.Tensor, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """codes int8 in [-8,7], scales = max(absmax, eps) / 7."""
    return _quantize_rowwise(self, eps, 7.0, -8, 7, False, "_quantize_int4_rowwise")


def _quantize_int2_rowwise(self: torch.Tensor, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """codes int8 in {-2,-1,0,1}, scales = max(absmax, eps) / 2."""
    return _quantize_rowwise(self, eps, 2.0, -2, 1, False, "_quantize_int2_rowwise")


def _quantize_binary_rowwise(self: torch.Tensor, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """codes int8 in {-1,+1} (x >= 0 -> +1), scales = max(absmax, eps)."""
    return _quantize_rowwise(self, eps, 1.0, -1, 1, True, "_quantize_binary_rowwise")


def _check_int_mm_operands(self, mat2):
    if self.dim() != 2 or mat2.dim() != 2:
        raise RuntimeError(f"_int_mm: expected two matrices but got {self.dim()}-D and {mat2.dim()}-D tensors")
    if self.size(1) != mat2.size(0):
        raise RuntimeError(f"_int_mm: cannot multiply a {self.size(0)} by {self.size(1)} matrix with a "
                           f"{mat2.size(0)} by {mat2.size(1)} matrix")
    if self.dtype not in (torch.int8, torch.uint8):
        raise RuntimeError("_int_mm: expected the left operand to be int8 or uint8")
    if mat2.dtype != torch.int8:
        raise RuntimeError("_int_mm: expected the right operand to be int8")


def _int_mm(self: torch.Tensor, mat2: torch.Tensor, *, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """C[M,N] int32 = self[M,K] (int8/uint8) @ mat2[K,N] (int8).

    The transposed view of a contiguous [N,K] weight (strides (1,K)) is consumed in place;
    any other layout of mat2 is made contiguous first.
    """
    _check_int_mm_operands(self, mat2)
    _require_device(self, "_int_mm")
    M, K = self.shape
    N = mat2.size(1)
    if out is not None:
        if out.dtype != torch.int32:
            raise RuntimeError("_int_mm: expected an int32 destination")
        if tuple(out.shape) != (M, N):
            out.resize_((M, N))
    dst = out if (out is not None and out.is_contiguous()) else torch.empty((M, N), dtype=torch.int32, device=self.device)
    if M and N:
        a = self.contiguous()
        if K and mat2.stride(0) == 1 and mat2.stride(1) == K:
            b, sbk, sbn = mat2, 1, K
        else:
            b = mat2.contiguous()
            sbk, sbn = N, 1
        lib = _lib.load()
        with torch.cuda.device(self.device):
            # a few hundred rows against a long K: slices of the k range meet in a scratch matrix (same bits)
            scratch_bytes = int(lib.tpq_int8_mm_workspace_bytes(M, N, K)) if (sbk == 1 and a.dtype == torch.int8) else 0
            if scratch_bytes:
                scratch = torch.empty(scratch_bytes // 4, dtype=torch.int32, device=self.device)
                _check(lib.tpq_int_mm_ws(_ptr(a), 0, _ptr(b), sbk, sbn, _ptr(dst), M, K, N, _ptr(scratch), scratch_bytes,
                                         _stream(self)))
            else:
                _check(lib.tpq_int_mm(_ptr(a), int(a.dtype == torch.uint8), _ptr(b), sbk, sbn, _ptr(dst),
                                      M, K, N, _stream(self)))
    if out is not None and dst is not out:
        out.copy_(dst)
    return out if out is not None else dst


def _int8_mm_rescale(out: torch.Tensor, row_scale: torch.Tensor, col_scale: torch.Tensor) -> torch.Tensor:
    """float32 result[m,n] = (float(out[m,n]) * row_scale[m]) * col_scale[n]."""
    if out.dim() != 2 or out.dtype != torch.int32:
        raise ValueError("_int8_mm_rescale(): expected a 2-D int32 output")
    _require_device(out, "_int8_mm_rescale")
    M, N = out.shape
    result = torch.empty((M, N), dtype=torch.float32, device=out.device)
    if M == 0 or N == 0:
        return result
    acc = out.contiguous()
    rs = row_scale.contiguous().to(torch.float32)
    cs = col_scale.contiguous().to(torch.float32)
    if rs.numel() != M or cs.numel() != N:
        raise ValueError("_int8_mm_rescale(): scale sizes do not match the output")
    with torch.cuda.device(out.device):
        _check(_lib.load().tpq_int8_mm_rescale(_ptr(acc), _ptr(rs), _ptr(cs), _ptr(result), M, N, _stream(out)))
    return result


def _quantized_weight_prepack(weight: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """int8 weight ``[N, K]`` -> (``packed`` int8 ``[N, ceil(K / 32) * 32]``, zero padded, ``offsets`` int64 ``[N]`` = row sums),
    the reference's ``_quantized_weight_prepack`` (p10/src/backend/cpu/QuantPacked.cpp:519-533).  One-time, tensor ops."""
    if weight.dim() != 2 or weight.dtype != torch.int8:
        raise TypeError("_quantized_weight_prepack: expected a 2-D int8 weight")
    _require_device(weight, "_quantized_weight_prepack")
    n, k = weight.shape
    packed = torch.zeros((n, (k + 31) // 32 * 32), dtype=torch.int8, device=weight.device)
    packed[:, :k] = weight
    return packed, weight.to(torch.int64).sum(1)


def _quantized_packed_run_linear(x_codes: torch.Tensor, x_scale: float, x_zero_point: int, packed: torch.Tensor,
                                 offsets: torch.Tensor, scales: torch.Tensor, zero_points: torch.Tensor,
                                 bias: Optional[torch.Tensor], in_features: int, relu: bool = False) -> torch.Tensor:
    """The linear, ``output_float=True`` form of the reference's ``_quantized_packed_run``
    (p10/src/backend/cpu/QuantPacked.cpp:420-516, 537-572) on the codes of a per-tensor quantized activation:
    ``fmaf(float(acc), float(x_scale) * scales[n], bias[n])`` with ``acc = x.w - xz off[n] - wz[n] sum(x) + K xz wz[n]``.
    x_codes ``[M, K]`` int8 or uint8; packed / offsets from ``_quantized_weight_prepack``; result float32 ``[M, N]``."""
    if x_codes.dim() != 2 or x_codes.dtype not in (torch.int8, torch.uint8):
        raise TypeError("_quantized_packed_run_linear: expected 2-D int8 or uint8 activation codes")
    if packed.dim() != 2 or packed.dtype != torch.int8:
        raise TypeError("_quantized_packed_run_linear: expected a 2-D int8 packed weight")
    m, k = x_codes.shape
    n = packed.size(0)
    if k != in_features or packed.size(1) < k:
        raise ValueError("_quantized_packed_run_linear: K dimension mismatch")
    if offsets.numel() != n or scales.numel() != n or zero_points.numel() != n or (bias is not None and bias.numel() != n):
        raise ValueError("_quantized_packed_run_linear: per-channel parameters must have one entry per output channel")
    _require_device(x_codes, "_quantized_packed_run_linear")
    out = torch.empty((m, n), dtype=torch.float32, device=x_codes.device)
    if m == 0 or n == 0:
        return out
    x, w = x_codes.contiguous(), packed.contiguous()
    off, zp = offsets.to(torch.int64).contiguous(), zero_points.to(torch.int64).contiguous()
    sc = scales.to(torch.float32).contiguous()
    b = None if bias is None else bias.to(torch.float32).contiguous()
    lib = _lib.load()
    unsigned = int(x.dtype == torch.uint8)
    with torch.cuda.device(x.device):
        need = int(lib.tpq_packed_linear_workspace_bytes(m, n, k, unsigned))
        ws = torch.empty(need, dtype=torch.uint8, device=x.device)
        _check(lib.tpq_packed_linear_float(_ptr(x), unsigned, float(x_scale), int(x_zero_point), _ptr(w), w.size(1), _ptr(off), _ptr(sc),
                                           _ptr(zp), _ptr(b), int(bool(relu)), _ptr(out), m, n, k, _ptr(ws), need, _stream(x)))
    return out


def int8_mm_dequant(A_i8: torch.Tensor, B_t_i8: torch.Tensor, row_scale: torch.Tensor, col_scale: torch.Tensor,
                    bias: Optional[torch.Tensor] = None, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """``_int_mm`` + ``_int8_mm_rescale`` (+ bias) in one launch.

    ``A_i8`` [M,K] int8, ``B_t_i8`` [N,K] int8, both contiguous; the result is
    ``cast((float(acc) * row_scale[m]) * col_scale[n] (+ bias[n]))``: the fp32 value the two
    reference ops produce, rounded once when ``out_dtype`` is a 16-bit float.
    """
    if A_i8.dim() != 2 or B_t_i8.dim() != 2 or A_i8.size(1) != B_t_i8.size(1):
        raise ValueError("int8_mm_dequant: expected A [M,K] and B_t [N,K]")
    if A_i8.dtype != torch.int8 or B_t_i8.dtype != torch.int8:
        raise TypeError("int8_mm_dequant: operands must be int8")
    if out_dtype not in _DT:
        raise TypeError("int8_mm_dequant: unsupported output dtype")
    _require_device(A_i8, "int8_mm_dequant")
    M, K = A_i8.shape
    N = B_t_i8.size(0)
    out = torch.empty((M, N), dtype=out_dtype, device=A_i8.device)
    if M == 0 or N == 0:
        return out
    a, w = A_i8.contiguous(), B_t_i8.contiguous()
    rs = row_scale.contiguous().to(torch.float32)
    cs = col_scale.contiguous().to(torch.float32)
    if rs.numel() != M or cs.numel() != N:
        raise ValueError("int8_mm_dequant: scale sizes do not match the output")
    b = None if bias is None else bias.contiguous().to(torch.float32)
    if b is not None and b.numel() != N:
        raise ValueError("int8_mm_dequant: bias must have one value per output channel")
    lib = _lib.load()
    with torch.cuda.device(a.device):
        # a few hundred rows against a long K: the library cuts the k range into slices that meet in an int32
        # scratch matrix (same bits as the single launch); it says for which shapes that pays
        scratch_bytes = int(lib.tpq_int8_mm_workspace_bytes(M, N, K))
        if scratch_bytes:
            scratch = torch.empty(scratch_bytes // 4, dtype=torch.int32, device=a.device)
            _check(lib.tpq_int8_mm_dequant_ws(_ptr(a), _ptr(w), _ptr(rs), _ptr(cs), _ptr(b), _ptr(out), _DT[out_dtype],
                                              M, N, K, _ptr(scratch), scratch_bytes, _stream(a)))
        else:
            _check(lib.tpq_int8_mm_dequant(_ptr(a), _ptr(w), _ptr(rs), _ptr(cs), _ptr(b), _ptr(out),
                                           _DT[out_dtype], M, N, K, _stream(a)))
    return out


_int4_workspaces = {}


def _int4_workspace(device: torch.device, m: int, n: int, k: int) -> torch.Tensor:
    """Zero-filled scratch buffer of the int4 kernels, one per (device, stream), grown on demand.
    The kernels leave the counters at the front of it zero again after every call."""
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    need = _lib.load().tpq_int4_mm_rows_workspace_bytes(m, n, k)
    ws = _int4_workspaces.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.zeros(need, dtype=torch.uint8, device=device)
        _int4_workspaces[key] = ws
    return ws


def _convert_weight_to_int4pack(self: torch.Tensor, innerKTiles: int) -> torch.Tensor:
    """int32 codes [N,K] (0..15) -> int32 [ceil(N/8), ceil(K/(16*innerKTiles)), 32, innerKTiles/2]."""
    if self.dim() != 2:
        raise ValueError("_convert_weight_to_int4pack(): expected 2-D codes [N,K]")
    if innerKTiles not in (2, 4, 8):
        raise ValueError("_convert_weight_to_int4pack(): innerKTiles must be 2, 4 or 8")
    N, K = self.shape
    if K % 2 != 0:
        raise ValueError("_convert_weight_to_int4pack(): K must be even")
    _require_device(self, "_convert_weight_to_int4pack")
    n_tiles = (N + 7) // 8
    k_super = (K + innerKTiles * 16 - 1) // (innerKTiles * 16)
    out = torch.empty((n_tiles, k_super, 32, innerKTiles // 2), dtype=torch.int32, device=self.device)
    if N == 0 or K == 0:
        return out
    codes = self.to(torch.int32).contiguous()
    with torch.cuda.device(self.device):
        _check(_lib.load().tpq_int4_pack(_ptr(codes), N, K, innerKTiles, _ptr(out), _stream(self)))
    return out


# Above this many activation rows _weight_int4pack_mm dequantises the weight and multiplies with the library's dense
# 16-bit tile kernel (tpq_dense_mm); below, the kernels that read the packed weight run (decode kernels up to 112 rows, a
# tiled kernel above).  Measured (us, packed-weight kernels / dense route including its dequantize pass of 21 us in
# float16 and 25 us in bfloat16 at K = 4096, N = 11008).  float16: K = 4096, N = 11008: 53 / 54 at 256 rows, 66 / 65 at
# 384, 71 / 68 at 512, 141 / 120 at 1024, 233 / 180 at 2048; K = N = 4096: 35 / 41 at 256, 61 / 38 at 384; K = N = 8192:
# 68 / 76 at 256, 114 / 97 at 384; K = 11008, N = 4096: 84 / 86 at 256, 150 / 92 at 384; K = 8192, N = 28672: 393 / 469
# at 768, 522 / 562 at 1024, 1012 / 875 at 2048.  bfloat16 pays ten vector operations per pair of weights for the dense
# weight's two roundings in the tiled kernel (float16: three packed ones), so it hands over earlier: K = 4096,
# N = 11008: 34 / 48 at 96, 51 / 48 at 128; K = N = 8192: 59 / 77 at 96, 96 / 79 at 128; K = 11008, N = 4096: 71 / 82 at
# 96, 127 / 87 at 128; K = 8192, N = 28672: 466 / 479 at 768, 623 / 565 at 1024.
INT4_PREFILL_ROWS = 256
INT4_PREFILL_ROWS_VERY_WIDE = 1024  # N >= 16384
INT4_PREFILL_ROWS_BF16 = 112
INT4_PREFILL_ROWS_BF16_VERY_WIDE = 768
# Between INT4_PREFILL_ROWS_BF16 and INT4_PREFILL_ROWS rows bfloat16 takes the tiled kernel where its estimate (1.4 times
# float16's, which is int4_gemm_plan of int4_gemm_kernel.h restated below: with a workspace that kernel deals K to
# slices when its tiles are few) is below the dense route's: 0.55 us per million weights for the dequantize pass and one
# round of tiles of the dense kernel.  Measured (us, dense / tiled, 128 and 255 rows): 4096 x 4096 38.4 / 23.0 and
# 41.6 / 33.9; 11008 -> 4096 89.8 / 42.8 and 92.5 / 71.1; 8192 x 8192 80.9 / 55.7 and 90.1 / 96.9; 4096 -> 11008
# 51.9 / 50.7 and 57.9 / 68.4.
def _int4_tiled_estimate_us(m: int, n: int, k: int) -> float:
    tiles = ((n + 63) // 64) * ((m + 127) // 128)

    def estimate(slices: int) -> float:
        per_unit = tiles * slices / 256.0
        rounds = 1.0 if per_unit <= 1.0 else 1.7 * int((per_unit + 1.999) / 2.0)
        return rounds * (5.0 + 7.2 * k / 1024.0 / slices) + (0.0 if slices == 1 else 1.6 + slices * m * n * 8.0 / 4e6)

    if m > 256 or k < 1024:
        return estimate(1)
    return min(estimate(s) for s in range(1, max(1, min(k // 128 // 4, 16)) + 1))


def _int4_dense_estimate_us(m: int, n: int, k: int) -> float:
    stages = k / 64.0
    short_rounds = -(-(((m + 127) // 128) * ((n + 127) // 128)) // 256)
    tall_rounds = -(-(((m + 255) // 256) * ((n + 127) // 128)) // 256)
    gemm = short_rounds * (stages * 690 + 8000) if short_rounds * 0.8 < tall_rounds else tall_rounds * (stages * 1080 + 9000)
    return 1.6 + 0.55e-6 * n * k + gemm / 2000.0


# float32 activations have no matrix-core decode kernel: the per-row kernel costs about 16 us a row at K = 4096,
# N = 11008 (71 us at 4 rows, 253 us at 16), the dense float32 route (the framework's GEMM) 95 us at 16 rows and 134 us at 64.
INT4_PREFILL_ROWS_F32 = 4


DENSE_F32_ROWS = 768


def _dense_mm(x: torch.Tensor, dense: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out = x @ dense.T`` behind the dequantise-then-multiply routes (QuantGemmKernels.cu:1339).

    K a multiple of 64 (float32: 32) runs the library's tile kernel; other K go to the framework's GEMM, and so do
    float32 activations below DENSE_F32_ROWS rows: the tile kernel takes 128 stages of four float32 MFMAs per fragment for
    K = 4096 whatever the row count (4096 -> 11008, us, library / framework: 8 rows 227 / 32, 512 rows 457 / 376, 2048 rows
    1362 / 1404 = 136 TFLOP/s of the 157 the matrix cores have for float32)."""
    m, k = x.shape
    n = dense.size(0)
    per_stage = 32 if x.dtype == torch.float32 else 64
    if (k % per_stage == 0 and k * (128 // per_stage) < (1 << 23) and x.data_ptr() % 16 == 0 and dense.data_ptr() % 16 == 0
            and (x.dtype != torch.float32 or m >= DENSE_F32_ROWS)):
        with torch.cuda.device(x.device):
            _check(_lib.load().tpq_dense_mm(_ptr(x), _DT[x.dtype], m, k, _ptr(dense), n, _ptr(out), _stream(x)))
        return out
    return torch.matmul(x, dense.t(), out=out)


def _int4_dequantize(packed: torch.Tensor, inner: int, n: int, k: int, group: int, sz: torch.Tensor) -> torch.Tensor:
    """Dense [N, K] weight in sz.dtype: T(code - 8) * scale + zero, product and sum each rounded to T."""
    dense = torch.empty((n, k), dtype=sz.dtype, device=packed.device)
    with torch.cuda.device(packed.device):
        _check(_lib.load().tpq_int4_dequantize(_ptr(packed), inner, n, k, group, _ptr(sz), _DT[sz.dtype], _ptr(dense),
                                               _stream(packed)))
    return dense


def _weight_int4pack_mm(self: torch.Tensor, mat2: torch.Tensor, qGroupSize: int,
                        qScaleAndZeros: torch.Tensor) -> torch.Tensor:
    """``self @ W.T`` with W dequantised per group: (code - 8) * scale + zero; result in self.dtype."""
    if mat2.dtype != torch.int32 or mat2.dim() != 4:
        raise TypeError("_weight_int4pack_mm(): packed weight must be 4-D int32 in the tensor-core B layout")
    if self.dim() != 2:
        raise ValueError("_weight_int4pack_mm(): expected 2-D activations [m,k]")
    if not self.is_floating_point():
        raise TypeError("_weight_int4pack_mm(): activations must be floating point")
    if qGroupSize not in (32, 64, 128):
        raise ValueError("_weight_int4pack_mm(): qGroupSize must be 32, 64 or 128")
    m, k = self.shape
    n_tiles, k_super, inner = mat2.size(0), mat2.size(1), mat2.size(3) * 2
    n = n_tiles * 8
    if mat2.size(2) != 32 or inner not in (2, 4, 8):
        raise ValueError("_weight_int4pack_mm(): packed weight layout is invalid")
    if k_super != (k + inner * 16 - 1) // (inner * 16):
        raise ValueError("_weight_int4pack_mm(): K dimension does not match packed B")
    groups = (k + qGroupSize - 1) // qGroupSize
    if qScaleAndZeros.dim() != 3 or tuple(qScaleAndZeros.shape) != (groups, n, 2):
        raise ValueError("_weight_int4pack_mm(): qScaleAndZeros must be [K/group, N, 2]")
    if self.dtype not in _DT:
        raise TypeError("_weight_int4pack_mm(): unsupported activation dtype")
    _require_device(self, "_weight_int4pack_mm")
    out = torch.empty((m, n), dtype=self.dtype, device=self.device)
    if m == 0 or n == 0 or k == 0:
        return out
    x = self.contiguous()
    w = mat2.contiguous()
    sz = qScaleAndZeros.to(self.dtype).contiguous()
    if self.dtype == torch.float32:
        prefill_rows = INT4_PREFILL_ROWS_F32
    elif self.dtype == torch.bfloat16:
        prefill_rows = INT4_PREFILL_ROWS_BF16_VERY_WIDE if n >= 16384 else INT4_PREFILL_ROWS_BF16
        if prefill_rows < m <= INT4_PREFILL_ROWS and k % 128 == 0 and 1.4 * _int4_tiled_estimate_us(m, n, k) < _int4_dense_estimate_us(m, n, k):
            prefill_rows = INT4_PREFILL_ROWS
    else:
        prefill_rows = INT4_PREFILL_ROWS_VERY_WIDE if n >= 16384 else INT4_PREFILL_ROWS
    if m > prefill_rows and inner == 2:
        # Many rows: what the reference does for every shape (QuantGemmKernels.cu:1296-1341) - dequantise
        # the weight to a dense matrix of the activation dtype, then one plain GEMM.  The decode
        # kernels read the packed weight once per 32 rows, which stops paying at this point.
        dense = _int4_dequantize(w, inner, n, k, qGroupSize, sz)
        return _dense_mm(x, dense, out)
    with torch.cuda.device(self.device):
        ws = _int4_workspace(self.device, m, n, k)
        _check(_lib.load().tpq_int4_mm_ws(_ptr(x), _DT[x.dtype], m, k, _ptr(w), inner, n, qGroupSize, _ptr(sz),
                                          _ptr(out), _ptr(ws), ws.numel(), _stream(self)))
    return out


def pack_ternary(codes: torch.Tensor) -> torch.Tensor:
    """int8 codes {-1,0,1} -> uint8, four per byte along the last dim (first code in bits 7..6)."""
    _require_device(codes, "pack_ternary")
    x = codes.to(torch.int8).contiguous()
    cols = x.shape[-1]
    rows = x.numel() // cols if cols else 0
    out = torch.empty((*x.shape[:-1], (cols + 3) // 4), dtype=torch.uint8, device=x.device)
    if rows and cols:
        with torch.cuda.device(x.device):
            _check(_lib.load().tpq_ternary_pack(_ptr(x), rows, cols, _ptr(out), _stream(x)))
    return out


def unpack_ternary(packed: torch.Tensor, columns: int) -> torch.Tensor:
    """uint8 packed -> int8 codes, sign-extending every 2-bit field; keeps the first `columns`."""
    _require_device(packed, "unpack_ternary")
    p = packed.contiguous()
    bytes_per_row = p.shape[-1]
    cols = min(int(columns), bytes_per_row * 4)
    rows = p.numel() // bytes_per_row if bytes_per_row else 0
    out = torch.empty((*p.shape[:-1], cols), dtype=torch.int8, device=p.device)
    if rows and cols:
        if (cols + 3) // 4 != bytes_per_row:
            p = p[..., : (cols + 3) // 4].contiguous()
        with torch.cuda.device(p.device):
            _check(_lib.load().tpq_ternary_unpack(_ptr(p), rows, cols, _ptr(out), _stream(p)))
    return out


def ternary_mm(x_i8: torch.Tensor, row_scale: torch.Tensor, packed: torch.Tensor, w_scale: float,
               in_features: int, bias: Optional[torch.Tensor] = None, out_dtype: torch.dtype = torch.float32,
               return_acc: bool = False):
    """``(float(x_i8 @ codes.T) * row_scale) * w_scale (+ bias)`` straight from the packed weight."""
    if x_i8.dim() != 2 or x_i8.dtype != torch.int8 or x_i8.size(1) != in_features:
        raise ValueError("ternary_mm: expected int8 activations [M, in_features]")
    if packed.dim() != 2 or packed.dtype != torch.uint8 or packed.size(1) != (in_features + 3) // 4:
        raise ValueError("ternary_mm: packed weight must be uint8 [N, ceil(in_features/4)]")
    if out_dtype not in _DT:
        raise TypeError("ternary_mm: unsupported output dtype")
    _require_device(x_i8, "ternary_mm")
    M, K = x_i8.shape
    N = packed.size(0)
    out = torch.empty((M, N), dtype=out_dtype, device=x_i8.device)
    acc = torch.empty((M, N), dtype=torch.int32, device=x_i8.device) if return_acc else None
    if M and N:
        x, p = x_i8.contiguous(), packed.contiguous()
        rs = row_scale.contiguous().to(torch.float32)
        if rs.numel() != M:
            raise ValueError("ternary_mm: one row scale per activation row expected")
        b = None if bias is None else bias.contiguous().to(torch.float32)
        lib = _lib.load()
        with torch.cuda.device(x.device):
            # prefill chunks against a long K: the library cuts K into splits that meet in an int32 scratch matrix
            # (same bits); it says for which shapes
            scratch_bytes = int(lib.tpq_ternary_mm_workspace_bytes(M, N, K))
            scratch = torch.empty(scratch_bytes // 4, dtype=torch.int32, device=x.device) if scratch_bytes else None
            _check(lib.tpq_ternary_mm_ws(_ptr(x), _ptr(rs), _ptr(p), float(w_scale), _ptr(b), M, N, K,
                                         _ptr(out), _DT[out_dtype], _ptr(acc), _ptr(scratch), scratch_bytes, _stream(x)))
    return (out, acc) if return_acc else out


# Above this many activation rows _weight_int8pack_mm dequantises and multiplies with the dense 16-bit tile kernel.
# Measured (fp16 / bf16 alike unless said, us, slabs of 32 rows on the decode kernels / dense route): K = 4096,
# N = 11008: 32 / 50 at 64 rows, 48 / 50 (bf16: 55 / 50) at 96, 62 / 51 at 128; K = N = 4096: 27 / 38 at 96, 37 / 39 at 128,
# 56 / 41 at 192; K = N = 8192: 58 / 78 at 64, 86 / 79 at 96; 11008 -> 4096: 58 / 83 at 64, 87 / 84 at 96; 8192 -> 28672:
# 202 / 249 at 64, 303 / 248 at 96.
INT8PACK_PREFILL_ROWS = 80
INT8PACK_PREFILL_ROWS_SHORT = 96  # K <= 4096
INT8PACK_PREFILL_ROWS_F32 = 24  # float32 activations (per-row kernel, the framework's GEMM): 64 / 89 us at 16 rows, 119 / 94 us at 32


def _int8pack_prefill_rows(N: int, K: int, dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return INT8PACK_PREFILL_ROWS_F32
    return INT8PACK_PREFILL_ROWS_SHORT if K <= 4096 else INT8PACK_PREFILL_ROWS


def _weight_int8pack_mm(self: torch.Tensor, mat2: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """``(self @ mat2.T) * scales``: activations [B,K] float, int8 weight [N,K], per-row scales [N];
    fp32 accumulation, result in the activation dtype (reference: QuantGemmKernels.cu:345-405)."""
    if mat2.dtype != torch.int8:
        raise TypeError("_weight_int8pack_mm(): weight must be QInt8")
    if self.dim() != 2 or mat2.dim() != 2 or scales.dim() != 1:
        raise ValueError("_weight_int8pack_mm(): expected 2-D activations [B,K], 2-D weight [N,K] and 1-D scales [N]")
    if self.dtype not in _DT:
        raise TypeError("_weight_int8pack_mm(): activations must be floating point")
    B, K = self.shape
    N = mat2.size(0)
    if mat2.size(1) != K:
        raise ValueError("_weight_int8pack_mm(): K dimension mismatch")
    if scales.size(0) != N:
        raise ValueError("_weight_int8pack_mm(): scales length mismatch")
    _require_device(self, "_weight_int8pack_mm")
    out = torch.empty((B, N), dtype=self.dtype, device=self.device)
    if B == 0 or N == 0 or K == 0:
        return out
    x, w = self.contiguous(), mat2.contiguous()
    sc = scales.to(torch.float32).contiguous()
    with torch.cuda.device(x.device):
        if B > _int8pack_prefill_rows(N, K, x.dtype):
            # Many rows: the decode kernel streams the weight once per 32 rows, which stops paying here.  One pass
            # writes the dense weight T(w * scale) and the dense tile kernel does the rest.
            dense = torch.empty((N, K), dtype=x.dtype, device=x.device)
            _check(_lib.load().tpq_int8pack_dequantize(_ptr(w), _ptr(sc), N, K, _DT[x.dtype], _ptr(dense), _stream(x)))
            return _dense_mm(x, dense, out)
        _check(_lib.load().tpq_weight_int8pack_mm(_ptr(x), _DT[x.dtype], B, K, _ptr(w), _ptr(sc), N, _ptr(out), _stream(x)))
    return out


def _convert_weight_to_int4pack_for_cpu(self: torch.Tensor, innerKTiles: int, *, block_cols: int = 64,
                                        half_split: bool = True) -> torch.Tensor:
    """int32 codes [N,K] -> the reference's CPU layout, uint8 [N, K/2] (default: the AVX-512 tier, whose bytes
    equal PyTorch's CPU pack), written by the GPU."""
    if self.dim() != 2 or self.dtype != torch.int32:
        raise ValueError("_convert_weight_to_int4pack_for_cpu(): expected 2-D int32 codes")
    _require_device(self, "_convert_weight_to_int4pack_for_cpu")
    N, K = self.shape
    out = torch.empty((N, K // 2), dtype=torch.uint8, device=self.device)
    codes = self.contiguous()
    with torch.cuda.device(self.device):
        _check(_lib.load().tpq_int4_pack_cpu_layout(_ptr(codes), N, K, int(block_cols), int(bool(half_split)), _ptr(out), _stream(self)))
    return out


def int4pack_cpu_to_device(packed_cpu: torch.Tensor, *, block_cols: int = 64, half_split: bool = True) -> torch.Tensor:
    """CPU-layout packed weight uint8 [N, K/2] -> device layout int32 [N/8, ceil(K/32), 32, 1]."""
    if packed_cpu.dim() != 2 or packed_cpu.dtype != torch.uint8:
        raise ValueError("int4pack_cpu_to_device(): expected a 2-D uint8 packed weight")
    _require_device(packed_cpu, "int4pack_cpu_to_device")
    N, K = packed_cpu.size(0), packed_cpu.size(1) * 2
    out = torch.empty((N // 8, (K + 31) // 32, 32, 1), dtype=torch.int32, device=packed_cpu.device)
    p = packed_cpu.contiguous()
    with torch.cuda.device(p.device):
        _check(_lib.load().tpq_int4_cpu_layout_to_device(_ptr(p), N, K, int(block_cols), int(bool(half_split)), _ptr(out), _stream(p)))
    return out


# ---- block-wise affine quantizer ----------------------------------------------------------------

# quantized dtype -> (storage tag, torch dtype of the code tensor, codes per byte).  The reference's
# quantized dtypes (p10 DType::QInt8 ... QUInt1x8) are named by string, or by the torch dtype of the
# same name where torch has one.
_AFFINE_STORAGE = {
    "qint8": (_lib.STORAGE_I8, torch.int8, 1),
    "quint8": (_lib.STORAGE_U8, torch.uint8, 1),
    "qint32": (_lib.STORAGE_I32, torch.int32, 1),
    "quint4x2": (_lib.STORAGE_U4X2, torch.uint8, 2),
    "quint2x4": (_lib.STORAGE_U2X4, torch.uint8, 4),
    "quint1x8": (_lib.STORAGE_U1X8, torch.uint8, 8),
}
_AFFINE_ALIASES = {torch.qint8: "qint8", torch.quint8: "quint8", torch.qint32: "qint32",
                   torch.quint4x2: "quint4x2", torch.quint2x4: "quint2x4"}
if hasattr(torch, "uint1"):
    _AFFINE_ALIASES[torch.uint1] = "quint1x8"


class PackedCodes:
    """Codes of a packed sub-byte dtype: ``shape`` logical elements, stored low bits first in the flat
    uint8 tensor ``data`` (element i in bits (i % pack) * bits of byte i // pack).  Stands in for the
    reference's tensors of dtype quint4x2 / quint2x4 / quint1x8, whose storage has the same bytes."""

    def __init__(self, data: torch.Tensor, shape, dtype: str):
        self.data, self.shape, self.dtype = data, tuple(shape), dtype

    @property
    def device(self):
        return self.data.device

    def untyped_bytes(self) -> torch.Tensor:
        return self.data


def _affine_dtype_name(dtype, op: str) -> str:
    name = _AFFINE_ALIASES.get(dtype, dtype)
    if name not in _AFFINE_STORAGE:
        raise TypeError(f"{op}(): expected a quantized dtype, got {dtype}")
    return name


def _affine_args(op, shape, block_size, scales, zero_points, device):
    import ctypes
    if len(block_size) != len(shape):
        raise ValueError(f"{op}(): block_size rank must match the input rank")
    if scales.device != device or (zero_points is not None and zero_points.numel() > 0 and zero_points.device != device):
        raise RuntimeError(f"{op}(): scales and zero_points must be on the input device")
    sc = scales.to(torch.float32).contiguous()
    zp = None
    if zero_points is not None and zero_points.numel() > 0:
        zp = zero_points.to(torch.float32).contiguous()
    arr = ctypes.c_int64 * max(len(shape), 1)
    return arr(*shape), arr(*[int(b) for b in block_size]), sc, zp


def quantize_affine(input: torch.Tensor, block_size, scales: torch.Tensor, zero_points: Optional[torch.Tensor],
                    dtype, quant_min: int, quant_max: int):
    """Block-wise affine quantization, ``clamp(rint(x * (1 / scale)) + zero_point)`` per block.

    Returns an int8 / uint8 / int32 tensor of the input's shape, or ``PackedCodes`` for the sub-byte
    dtypes.  Reference: ``quantize_affine`` (config/native_functions.yaml:5308,
    p10/src/backend/cpu/QuantKernels.cpp:579-774).
    """
    import ctypes
    name = _affine_dtype_name(dtype, "quantize_affine")
    tag, code_dtype, pack = _AFFINE_STORAGE[name]
    _require_device(input, "quantize_affine")
    if input.dtype not in _DT:
        input = input.to(torch.float32)
    x = input.contiguous()
    sizes, blocks, sc, zp = _affine_args("quantize_affine", tuple(x.shape), block_size, scales, zero_points, x.device)
    numel = x.numel()
    if pack == 1:
        out = torch.empty(x.shape, dtype=code_dtype, device=x.device)
    else:
        out = torch.empty(((numel + pack - 1) // pack,), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        _check(_lib.load().tpq_quantize_affine(_ptr(x), _DT[x.dtype], x.dim(), ctypes.cast(sizes, ctypes.c_void_p),
                                               ctypes.cast(blocks, ctypes.c_void_p), _ptr(sc), sc.numel(), _ptr(zp),
                                               0 if zp is None else zp.numel(), tag, int(quant_min), int(quant_max),
                                               _ptr(out), _stream(x)))
    return out if pack == 1 else PackedCodes(out, x.shape, name)


def dequantize_affine(input, block_size, scales: torch.Tensor, zero_points: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 ``(code - zero_point) * scale`` per block; the inverse map of ``quantize_affine``.

    ``input`` is an int8 / uint8 / int32 code tensor or ``PackedCodes``.  Reference:
    ``dequantize_affine`` (config/native_functions.yaml:5314, p10/src/backend/cpu/QuantKernels.cpp:776-990).
    """
    import ctypes
    if isinstance(input, PackedCodes):
        name, codes, shape = input.dtype, input.data, input.shape
    else:
        by_dtype = {torch.int8: "qint8", torch.uint8: "quint8", torch.int32: "qint32"}
        if not isinstance(input, torch.Tensor) or input.dtype not in by_dtype:
            raise TypeError(f"dequantize_affine(): expected a quantized tensor, got {getattr(input, 'dtype', type(input))}")
        name, codes, shape = by_dtype[input.dtype], input.contiguous(), tuple(input.shape)
    tag = _AFFINE_STORAGE[name][0]
    _require_device(codes, "dequantize_affine")
    sizes, blocks, sc, zp = _affine_args("dequantize_affine", shape, block_size, scales, zero_points, codes.device)
    out = torch.empty(shape, dtype=torch.float32, device=codes.device)
    with torch.cuda.device(codes.device):
        _check(_lib.load().tpq_dequantize_affine(_ptr(codes), tag, len(shape), ctypes.cast(sizes, ctypes.c_void_p),
                                                 ctypes.cast(blocks, ctypes.c_void_p), _ptr(sc), sc.numel(), _ptr(zp),
                                                 0 if zp is None else zp.numel(), _ptr(out), _stream(codes)))
    return out


# ---- packed n-bit weight-only linear (int2 / intx / binary modules) ------------------------------

# above this many activation rows the weight is dequantised once for the dense 16-bit tile kernel (measured, 2 and 4
# bits, float16 and bfloat16 alike, us, decode kernel / dense route: K = 4096, N = 11008: 34 / 58 at 32 rows, 51 / 58 at
# 48, 68 / 58 at 64; K = N = 4096: 29 / 42 at 64, 42 / 42 at 96, 56 / 42 at 128)
LOWBIT_PREFILL_ROWS = 56
LOWBIT_PREFILL_ROWS_SMALL = 80  # N K <= 2^24
LOWBIT_PREFILL_ROWS_F32 = 40  # float32 activations (per-row kernel): 144 / 165 us at 32 rows, 278 / 192 us at 64 (K = 4096, N = 11008)


def _lowbit_codes(t: torch.Tensor, what: str) -> torch.Tensor:
    _require_device(t, what)
    if t.dtype not in (torch.uint8, torch.int8):
        t = t.to(torch.uint8)
    return t.contiguous().view(torch.uint8)


def pack_lowbit(codes: torch.Tensor, bits: int, lsb_first: bool = False) -> torch.Tensor:
    """uint8 [..., ceil(cols / (8 // bits))]: ``8 // bits`` codes per byte, the first in the most
    significant bits (``pack_intx``) or, ``lsb_first``, code i in bit i (``pack_binary``)."""
    if not 1 <= bits <= 8:
        raise ValueError(f"bits must be in [1, 8], got {bits}")
    c = _lowbit_codes(codes, "pack_lowbit")
    cols = c.shape[-1]
    rows = c.numel() // cols if cols else 0
    per_byte = 8 // bits
    out = torch.empty((*c.shape[:-1], (cols + per_byte - 1) // per_byte), dtype=torch.uint8, device=c.device)
    with torch.cuda.device(c.device):
        _check(_lib.load().tpq_lowbit_pack(_ptr(c), bits, int(lsb_first), rows, cols, _ptr(out), _stream(c)))
    return out


def unpack_lowbit(packed: torch.Tensor, bits: int, columns: int, lsb_first: bool = False) -> torch.Tensor:
    """uint8 codes [..., columns] of a tensor written by ``pack_lowbit``."""
    if not 1 <= bits <= 8:
        raise ValueError(f"bits must be in [1, 8], got {bits}")
    p = _lowbit_codes(packed, "unpack_lowbit")
    per_byte = 8 // bits
    if p.shape[-1] != (columns + per_byte - 1) // per_byte:
        raise ValueError(f"unpack: {p.shape[-1]} bytes per row do not hold {columns} {bits}-bit codes")
    rows = p.numel() // p.shape[-1] if p.shape[-1] else 0
    out = torch.empty((*p.shape[:-1], columns), dtype=torch.uint8, device=p.device)
    with torch.cuda.device(p.device):
        _check(_lib.load().tpq_lowbit_unpack(_ptr(p), bits, int(lsb_first), rows, columns, _ptr(out), _stream(p)))
    return out


def _lowbit_operands(packed, bits, columns, scales_and_zeros, what):
    _require_device(packed, what)
    if packed.dim() != 2 or packed.dtype != torch.uint8:
        raise TypeError(f"{what}: expected a 2-D uint8 packed weight")
    per_byte = 8 // bits
    if packed.shape[1] != (columns + per_byte - 1) // per_byte:
        raise ValueError(f"{what}: {packed.shape[1]} bytes per row do not hold {columns} {bits}-bit codes")
    n = packed.shape[0]
    if scales_and_zeros.dim() != 3 or scales_and_zeros.shape[1] != n or scales_and_zeros.shape[2] != 2 or scales_and_zeros.shape[0] < 1:
        raise ValueError(f"{what}: scales_and_zeros must be [K / groupsize, N, 2]")
    if columns % scales_and_zeros.shape[0]:
        raise ValueError(f"{what}: K={columns} must be divisible by the number of groups {scales_and_zeros.shape[0]}")
    return packed.contiguous(), scales_and_zeros.to(torch.float32).contiguous(), n, columns // scales_and_zeros.shape[0]


def _lowbit_dequantize(packed, bits, columns, scales_and_zeros, dtype=torch.float32, lsb_first=False) -> torch.Tensor:
    """Dense [N, K] weight ``(code - zero) * scale`` of ``dtype`` (``_dequantize_intx``)."""
    w, sz, n, group = _lowbit_operands(packed, bits, columns, scales_and_zeros, "_lowbit_dequantize")
    out = torch.empty((n, columns), dtype=dtype, device=w.device)
    with torch.cuda.device(w.device):
        _check(_lib.load().tpq_lowbit_dequantize(_ptr(w), bits, int(lsb_first), n, columns, group, _ptr(sz), _DT[dtype],
                                                 _ptr(out), _stream(w)))
    return out


def _lowbit_mm(input: torch.Tensor, packed: torch.Tensor, bits: int, columns: int, scales_and_zeros: torch.Tensor,
               bias: Optional[torch.Tensor] = None, lsb_first: bool = False) -> torch.Tensor:
    """``input @ dequantize(packed).T (+ bias)`` for a packed n-bit weight, without the dense weight
    (``_intx_mm`` / ``_int2_mm`` / ``_binary_mm`` of the reference).  input [M, K] f32 / f16 / bf16."""
    if input.dim() != 2 or input.shape[1] != columns:
        raise ValueError(f"_lowbit_mm: expected activations [M, {columns}]")
    if input.dtype not in _DT:
        raise TypeError("_lowbit_mm: activations must be float32, float16 or bfloat16")
    _require_device(input, "_lowbit_mm")
    w, sz, n, group = _lowbit_operands(packed, bits, columns, scales_and_zeros, "_lowbit_mm")
    x = input.contiguous()
    m = x.shape[0]
    b = None if bias is None else bias.to(torch.float32).contiguous()
    if m > (LOWBIT_PREFILL_ROWS_F32 if x.dtype == torch.float32 else LOWBIT_PREFILL_ROWS_SMALL if n * columns <= (1 << 24) else LOWBIT_PREFILL_ROWS):
        dense = _lowbit_dequantize(w, bits, columns, sz, x.dtype, lsb_first)
        out = _dense_mm(x, dense, torch.empty((m, n), dtype=x.dtype, device=x.device))
        return out if b is None else out + b.to(out.dtype)
    out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        _check(_lib.load().tpq_lowbit_mm(_ptr(x), _DT[x.dtype], m, columns, _ptr(w), bits, int(lsb_first), n, group,
                                         _ptr(sz), _ptr(b), _ptr(out), _stream(x)))
    return out


# ---- fusions around the int4 decode matmul (MLP of a decoder layer) -------------------------------

def _fused_int4_check(x, packed, group, sz, what):
    """Shape, layout and extent checks of one (activations, packed weight, scales) triple; host only."""
    if packed.dtype != torch.int32 or packed.dim() != 4 or packed.size(2) != 32:
        raise TypeError(f"{what}: packed weight must be 4-D int32 in the tensor-core B layout")
    if x.dim() != 2 or x.dtype not in _DT:
        raise ValueError(f"{what}: expected 2-D float activations [m,k]")
    if group not in (32, 64, 128):
        raise ValueError(f"{what}: qGroupSize must be 32, 64 or 128")
    inner, n, k = packed.size(3) * 2, packed.size(0) * 8, x.shape[1]
    if inner not in (2, 4, 8):
        raise ValueError(f"{what}: packed weight layout is invalid")
    # the kernels only receive pointers: a packed weight that covers fewer k than the activations would be read
    # past its end, so the extent is checked here, as _weight_int4pack_mm does
    if packed.size(1) != (k + inner * 16 - 1) // (inner * 16):
        raise ValueError(f"{what}: K dimension does not match packed B")
    if sz.dim() != 3 or tuple(sz.shape) != ((k + group - 1) // group, n, 2):
        raise ValueError(f"{what}: qScaleAndZeros must be [K/group, N, 2]")
    return inner, n


def _fused_int4_operands(x, packed, group, sz, what):
    inner, n = _fused_int4_check(x, packed, group, sz, what)
    _require_device(x, what)
    return x.contiguous(), packed.contiguous(), sz.to(x.dtype).contiguous(), inner, n


def int4pack_mm_add(input: torch.Tensor, mat2: torch.Tensor, qGroupSize: int, qScaleAndZeros: torch.Tensor,
                    residual: torch.Tensor) -> torch.Tensor:
    """``residual + _weight_int4pack_mm(input, mat2, qGroupSize, qScaleAndZeros)`` in one launch, rounded
    where the two separate ops round.  Shapes the fused kernel does not take run the two ops."""
    x, w, sz, inner, n = _fused_int4_operands(input, mat2, qGroupSize, qScaleAndZeros, "int4pack_mm_add")
    m, k = x.shape
    if tuple(residual.shape) != (m, n) or residual.dtype != x.dtype:
        raise ValueError("int4pack_mm_add: residual must be [m, n] of the activation dtype")
    out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    if m == 0 or n == 0:
        return out
    r = residual.contiguous()
    with torch.cuda.device(x.device):
        status = _lib.load().tpq_int4_mm_add(_ptr(x), _DT[x.dtype], m, k, _ptr(w), inner, n, qGroupSize, _ptr(sz), _ptr(r),
                                             _ptr(out), _stream(x))
    if status == _lib.TPQ_ERR_UNSUPPORTED:
        return r + _weight_int4pack_mm(x, w, qGroupSize, sz)
    _check(status)
    return out


def rms_norm(input: torch.Tensor, weight: Optional[torch.Tensor] = None, eps: float = 1e-5) -> torch.Tensor:
    """The reference's ``rms_norm`` over the last dimension (native op ``rms_norm``, config/native_functions.yaml:5962;
    tensorplay/nn/functional.py:2350-2372): fp32 compute, ``(x * (1 / sqrt(mean(x^2) + eps))) * weight`` rounded once
    to the input dtype.  One launch; the fused entry points below fall back to it for the shapes they are not built for."""
    _require_device(input, "rms_norm()")
    if input.dim() < 1:
        raise ValueError("rms_norm(): expected at least one dimension")
    if input.dtype not in _DT:
        raise TypeError(f"rms_norm(): unsupported dtype {input.dtype}")
    k = input.shape[-1]
    if weight is not None:
        _require_device(weight, "rms_norm()")
        if weight.dim() != 1 or weight.numel() != k:
            raise ValueError("rms_norm(): weight must have the size of the last dimension")
        if weight.dtype != input.dtype:
            weight = weight.to(input.dtype)
        weight = weight.contiguous()
    x = input.contiguous()
    out = torch.empty_like(x)
    m = x.numel() // k if k else 0
    if m == 0 or k == 0:
        return out
    with torch.cuda.device(x.device):
        _check(_lib.load().tpq_rms_norm(_ptr(x), _DT[x.dtype], m, k, _ptr(weight), float(eps),
                                        _ptr(out), _stream(x)))
    return out


def _norm_operand(x: torch.Tensor, norm_weight: torch.Tensor, what: str) -> torch.Tensor:
    if norm_weight.dim() != 1 or norm_weight.numel() != x.shape[1] or norm_weight.dtype != x.dtype or norm_weight.device != x.device:
        raise ValueError(f"{what}: norm_weight must be [k] of the activation dtype, on the activations' device")
    return norm_weight.contiguous()


def int4pack_mm_multi(input: torch.Tensor, mats, qGroupSize: int, scales_and_zeros, norm_weight: Optional[torch.Tensor] = None,
                      eps: float = 1e-5) -> list:
    """``[_weight_int4pack_mm(input, w, qGroupSize, sz) for w, sz in zip(mats, scales_and_zeros)]`` with one launch
    per 16 rows for up to four weights (q, k, v of a decoder layer).  Shapes the fused kernel does not take, and more
    than four weights, run the separate op.  With ``norm_weight`` the products are taken of ``rms_norm(input,
    norm_weight, eps)``, normalized inside the same launch where the kernel is built for it."""
    mats, scales_and_zeros = list(mats), list(scales_and_zeros)
    if len(mats) != len(scales_and_zeros) or not mats:
        raise ValueError("int4pack_mm_multi: one qScaleAndZeros per packed weight, at least one weight")
    for w, sz in zip(mats, scales_and_zeros):
        _fused_int4_check(input, w, qGroupSize, sz, "int4pack_mm_multi")
    ops = [_fused_int4_operands(input, w, qGroupSize, sz, "int4pack_mm_multi") for w, sz in zip(mats, scales_and_zeros)]
    x = ops[0][0]
    m, k = x.shape

    g = None if norm_weight is None else _norm_operand(x, norm_weight, "int4pack_mm_multi")

    def separate():
        xn = x if g is None else rms_norm(x, g, eps)
        return [_weight_int4pack_mm(xn, w, qGroupSize, sz) for _, w, sz, _, _ in ops]

    if len(ops) > 4 or len({inner for _, _, _, inner, _ in ops}) != 1 or x.dtype == torch.float32:
        return separate()
    outs = [torch.empty((m, n), dtype=x.dtype, device=x.device) for _, _, _, _, n in ops]
    if m == 0:
        return outs
    count = len(ops)
    packed = (ctypes.c_void_p * count)(*[_ptr(w) for _, w, _, _, _ in ops])
    szs = (ctypes.c_void_p * count)(*[_ptr(sz) for _, _, sz, _, _ in ops])
    ys = (ctypes.c_void_p * count)(*[_ptr(o) for o in outs])
    widths = (ctypes.c_int64 * count)(*[n for _, _, _, _, n in ops])
    with torch.cuda.device(x.device):
        if g is None:
            status = _lib.load().tpq_int4_mm_multi(_ptr(x), _DT[x.dtype], m, k, count, ctypes.cast(packed, ctypes.c_void_p), ops[0][3],
                                                   ctypes.cast(widths, ctypes.c_void_p), qGroupSize, ctypes.cast(szs, ctypes.c_void_p),
                                                   ctypes.cast(ys, ctypes.c_void_p), _stream(x))
        else:
            status = _lib.load().tpq_int4_mm_multi_norm(_ptr(x), _DT[x.dtype], m, k, _ptr(g), float(eps), count,
                                                        ctypes.cast(packed, ctypes.c_void_p), ops[0][3],
                                                        ctypes.cast(widths, ctypes.c_void_p), qGroupSize,
                                                        ctypes.cast(szs, ctypes.c_void_p), ctypes.cast(ys, ctypes.c_void_p), _stream(x))
    if status == _lib.TPQ_ERR_UNSUPPORTED:
        return separate()
    _check(status)
    return outs


def int4pack_mm_swiglu(input: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, qGroupSize: int,
                       gate_scale_and_zeros: torch.Tensor, up_scale_and_zeros: torch.Tensor,
                       norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-5) -> torch.Tensor:
    """``silu_mul(_weight_int4pack_mm(input, gate, ...), _weight_int4pack_mm(input, up, ...))`` in one launch
    (the reference's ``silu_mul``: gate * sigmoid(gate) * up in float32, rounded once).  Shapes the fused kernel
    does not take run the separate ops.  With ``norm_weight`` the input is ``rms_norm(input, norm_weight, eps)``,
    normalized inside the same launch where the kernel is built for it."""
    _fused_int4_check(input, gate, qGroupSize, gate_scale_and_zeros, "int4pack_mm_swiglu")
    _fused_int4_check(input, up, qGroupSize, up_scale_and_zeros, "int4pack_mm_swiglu")
    x, wg, szg, inner, n = _fused_int4_operands(input, gate, qGroupSize, gate_scale_and_zeros, "int4pack_mm_swiglu")
    _, wu, szu, inner_u, n_u = _fused_int4_operands(input, up, qGroupSize, up_scale_and_zeros, "int4pack_mm_swiglu")
    if (inner_u, n_u) != (inner, n) or wu.shape != wg.shape:
        raise ValueError("int4pack_mm_swiglu: gate and up must have the same packed shape")
    m, k = x.shape
    out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    if m == 0 or n == 0:
        return out
    nw = None if norm_weight is None else _norm_operand(x, norm_weight, "int4pack_mm_swiglu")
    with torch.cuda.device(x.device):
        if nw is None:
            status = _lib.load().tpq_int4_mm_swiglu(_ptr(x), _DT[x.dtype], m, k, _ptr(wg), _ptr(wu), inner, n, qGroupSize, _ptr(szg),
                                                    _ptr(szu), _ptr(out), _stream(x))
        else:
            status = _lib.load().tpq_int4_mm_swiglu_norm(_ptr(x), _DT[x.dtype], m, k, _ptr(nw), float(eps), _ptr(wg), _ptr(wu), inner, n,
                                                         qGroupSize, _ptr(szg), _ptr(szu), _ptr(out), _stream(x))
    if status == _lib.TPQ_ERR_UNSUPPORTED:
        xn = x if nw is None else rms_norm(x, nw, eps)
        g = _weight_int4pack_mm(xn, wg, qGroupSize, szg).float()
        u = _weight_int4pack_mm(xn, wu, qGroupSize, szu).float()
        return (g * torch.sigmoid(g) * u).to(x.dtype)
    _check(status)
    return out
