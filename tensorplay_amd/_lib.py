"""Loads ``libtpq_gfx950.so`` and declares the C ABI of ``include/tpq.h`` for ctypes.

The library is required: if it has not been built, loading raises with the
command that builds it.  There is no CPU fallback.
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtpq_gfx950.so")

TPQ_OK, TPQ_ERR_INVALID_VALUE, TPQ_ERR_INVALID_TYPE, TPQ_ERR_RUNTIME, TPQ_ERR_UNSUPPORTED = range(5)
F32, F16, BF16 = 0, 1, 2
STORAGE_I8, STORAGE_U8, STORAGE_I32, STORAGE_U4X2, STORAGE_U2X4, STORAGE_U1X8 = range(6)

_i64, _int, _f32, _ptr = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p

# name -> argument types, in the order of include/tpq.h
SIGNATURES = {
    "tpq_abi_version": [],
    "tpq_quantize_rowwise": [_ptr, _int, _i64, _i64, _f32, _f32, _int, _int, _int, _ptr, _ptr, _ptr],
    "tpq_int_mm": [_ptr, _int, _ptr, _i64, _i64, _ptr, _i64, _i64, _i64, _ptr],
    "tpq_int8_mm_rescale": [_ptr, _ptr, _ptr, _ptr, _i64, _i64, _ptr],
    "tpq_int8_mm_dequant": [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _int, _i64, _i64, _i64, _ptr],
    "tpq_int8_mm_workspace_bytes": [_i64, _i64, _i64],
    "tpq_int_mm_ws": [_ptr, _int, _ptr, _i64, _i64, _ptr, _i64, _i64, _i64, _ptr, _i64, _ptr],
    "tpq_int8_mm_dequant_ws": [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _int, _i64, _i64, _i64, _ptr, _i64, _ptr],
    "tpq_int8_mm_noalloc_max_bytes": [],
    "tpq_int8_mm_dequant_noalloc": [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _int, _i64, _i64, _i64, _ptr],
    "tpq_int4_pack": [_ptr, _i64, _i64, _int, _ptr, _ptr],
    "tpq_int4_mm": [_ptr, _int, _i64, _i64, _ptr, _int, _i64, _i64, _ptr, _ptr, _ptr],
    "tpq_int4_mm_ws": [_ptr, _int, _i64, _i64, _ptr, _int, _i64, _i64, _ptr, _ptr, _ptr, ctypes.c_size_t, _ptr],
    "tpq_int4_mm_workspace_bytes": [_i64],
    "tpq_int4_mm_rows_workspace_bytes": [_i64, _i64, _i64],
    "tpq_ternary_pack": [_ptr, _i64, _i64, _ptr, _ptr],
    "tpq_ternary_unpack": [_ptr, _i64, _i64, _ptr, _ptr],
    "tpq_ternary_mm": [_ptr, _ptr, _ptr, _f32, _ptr, _i64, _i64, _i64, _ptr, _int, _ptr, _ptr],
    "tpq_ternary_mm_workspace_bytes": [_i64, _i64, _i64],
    "tpq_ternary_mm_ws": [_ptr, _ptr, _ptr, _f32, _ptr, _i64, _i64, _i64, _ptr, _int, _ptr, _ptr, _i64, _ptr],
    "tpq_int4_mm_add": [_ptr, _int, _i64, _i64, _ptr, _int, _i64, _i64, _ptr, _ptr, _ptr, _ptr],
    "tpq_int4_mm_swiglu": [_ptr, _int, _i64, _i64, _ptr, _ptr, _int, _i64, _i64, _ptr, _ptr, _ptr, _ptr],
    "tpq_int4_mm_multi": [_ptr, _int, _i64, _i64, _int, _ptr, _int, _ptr, _i64, _ptr, _ptr, _ptr],
    "tpq_int4_mm_swiglu_norm": [_ptr, _int, _i64, _i64, _ptr, _f32, _ptr, _ptr, _int, _i64, _i64, _ptr, _ptr, _ptr, _ptr],
    "tpq_rms_norm": [_ptr, _int, _i64, _i64, _ptr, _f32, _ptr, _ptr],
    "tpq_dense_mm": [_ptr, _int, _i64, _i64, _ptr, _i64, _ptr, _ptr],
    "tpq_packed_linear_workspace_bytes": [_i64, _i64, _i64, _int],
    "tpq_packed_linear_float": [_ptr, _int, ctypes.c_double, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _int, _ptr, _i64, _i64, _i64, _ptr,
                                ctypes.c_size_t, _ptr],
    "tpq_int4_mm_multi_norm": [_ptr, _int, _i64, _i64, _ptr, _f32, _int, _ptr, _int, _ptr, _i64, _ptr, _ptr, _ptr],
    "tpq_int4_dequantize": [_ptr, _int, _i64, _i64, _i64, _ptr, _int, _ptr, _ptr],
    "tpq_int4_pack_cpu_layout": [_ptr, _i64, _i64, _int, _int, _ptr, _ptr],
    "tpq_int4_cpu_layout_to_device": [_ptr, _i64, _i64, _int, _int, _ptr, _ptr],
    "tpq_weight_int8pack_mm": [_ptr, _int, _i64, _i64, _ptr, _ptr, _i64, _ptr, _ptr],
    "tpq_int8pack_dequantize": [_ptr, _ptr, _i64, _i64, _int, _ptr, _ptr],
    "tpq_quantize_affine": [_ptr, _int, _int, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _int, _i64, _i64, _ptr, _ptr],
    "tpq_lowbit_mm": [_ptr, _int, _i64, _i64, _ptr, _int, _int, _i64, _i64, _ptr, _ptr, _ptr, _ptr],
    "tpq_lowbit_dequantize": [_ptr, _int, _int, _i64, _i64, _i64, _ptr, _int, _ptr, _ptr],
    "tpq_lowbit_pack": [_ptr, _int, _int, _i64, _i64, _ptr, _ptr],
    "tpq_lowbit_unpack": [_ptr, _int, _int, _i64, _i64, _ptr, _ptr],
    "tpq_dequantize_affine": [_ptr, _int, _int, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _ptr],
}

_lib = None


def load() -> ctypes.CDLL:
    """Return the loaded kernel library (loading it on first use)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m tensorplay_amd.build` "
            "(hipcc --offload-arch=gfx950). There is no fallback implementation."
        )
    # torch first: its bundled HIP runtime (soname libamdhip64.so.7) must be the one in the
    # process, so that device pointers and streams are shared with the tensors we are handed.
    import torch  # noqa: F401

    _lib = bind(LIB_PATH)
    return _lib


def bind(path: str) -> ctypes.CDLL:
    """Opens a build of the kernel library and declares the operators' signatures on it."""
    lib = ctypes.CDLL(path)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = ctypes.c_size_t if name.endswith("_bytes") else _int
    lib.tpq_last_error.argtypes = []
    lib.tpq_last_error.restype = ctypes.c_char_p
    return lib


def last_error() -> str:
    return load().tpq_last_error().decode("utf-8", "replace")
