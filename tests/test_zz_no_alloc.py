"""The allocation-free entry point tpq_int8_mm_dequant_noalloc, called through the C ABI.

Its slice matrices live in a buffer built into the library, so the check is against tpq_int8_mm_dequant_ws with a
caller-allocated workspace (bit-exact: both add the same exact int32 partial sums) and against the oracle's
int32 product + rescale.  Two calls in a row, the second on a smaller problem, because every call on a GPU reuses
the same buffer and finds the previous call's contents in it.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from gpu_util import DEV

pytestmark = pytest.mark.gpu

_DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _operands(seed, M, N, K, with_bias):
    rng = np.random.default_rng(seed)
    a = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    w = rng.integers(-128, 128, size=(N, K)).astype(np.int8)
    rs = rng.uniform(0.005, 0.02, M).astype(np.float32)
    cs = rng.uniform(0.0005, 0.002, N).astype(np.float32)
    bias = rng.normal(0, 0.01, N).astype(np.float32) if with_bias else None
    return a, w, rs, cs, bias


def _run_pair(lib, M, N, K, out_dtype, with_bias, seed):
    from tensorplay_amd import _lib

    a, w, rs, cs, bias = _operands(seed, M, N, K, with_bias)
    da, dw, drs, dcs = (torch.from_numpy(v).to(DEV) for v in (a, w, rs, cs))
    db = torch.from_numpy(bias).to(DEV) if with_bias else None
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    need = lib.tpq_int8_mm_workspace_bytes(M, N, K)
    assert need > 0, "the shape must be one that cuts the k range into slices"
    assert need <= lib.tpq_int8_mm_noalloc_max_bytes()

    want = torch.full((M, N), 7, dtype=out_dtype, device=DEV)
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    rc = lib.tpq_int8_mm_dequant_ws(_ptr(da), _ptr(dw), _ptr(drs), _ptr(dcs), _ptr(db), _ptr(want), _DT[out_dtype], M, N, K,
                                    _ptr(ws), need, stream)
    assert rc == 0, _lib.last_error()

    got = torch.full((M, N), 9, dtype=out_dtype, device=DEV)
    rc = lib.tpq_int8_mm_dequant_noalloc(_ptr(da), _ptr(dw), _ptr(drs), _ptr(dcs), _ptr(db), _ptr(got), _DT[out_dtype], M, N, K, stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)), f"noalloc differs from _ws at {M}x{N}x{K}"

    if out_dtype == torch.float32:  # and both equal the oracle, bit for bit
        ref = oracle.int8_mm_rescale(oracle.int_mm(a, w.T), rs, cs)
        if with_bias:
            ref = (ref + bias[None, :]).astype(np.float32)
        np.testing.assert_array_equal(got.cpu().numpy(), ref)


def test_noalloc_equals_workspace_entry_point_two_calls_in_a_row():
    from tensorplay_amd import _lib

    lib = _lib.load()
    print("noalloc: 300x264x8192 f32 then 130x200x4096 f32", flush=True)
    _run_pair(lib, 300, 264, 8192, torch.float32, True, 1)   # first call: fills the built-in buffer
    _run_pair(lib, 130, 200, 4096, torch.float32, False, 2)  # second, smaller: the buffer still holds the first call's sums
    _run_pair(lib, 300, 264, 8192, torch.bfloat16, True, 3)
    _run_pair(lib, 132, 128, 4608, torch.float16, False, 4)


def test_noalloc_rejects_what_does_not_fit_and_passes_on_what_needs_no_scratch():
    from tensorplay_amd import _lib

    lib = _lib.load()
    limit = lib.tpq_int8_mm_noalloc_max_bytes()
    assert limit == 16 << 20
    M, N, K = 256, 4096, 11008   # 32 tiles, 86 stages -> 8 slices of 256 x 4096 int32 = 32 MiB
    need = lib.tpq_int8_mm_workspace_bytes(M, N, K)
    assert need > limit
    rc = lib.tpq_int8_mm_dequant_noalloc(None, None, None, None, None, None, 0, M, N, K, None)
    assert rc == _lib.TPQ_ERR_INVALID_VALUE and "scratch" in _lib.last_error()

    # a shape that uses no slices runs as the plain entry point
    M, N, K = 16, 256, 512
    assert lib.tpq_int8_mm_workspace_bytes(M, N, K) == 0
    a, w, rs, cs, _ = _operands(5, M, N, K, False)
    da, dw, drs, dcs = (torch.from_numpy(v).to(DEV) for v in (a, w, rs, cs))
    got = torch.empty((M, N), dtype=torch.float32, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.tpq_int8_mm_dequant_noalloc(_ptr(da), _ptr(dw), _ptr(drs), _ptr(dcs), None, _ptr(got), 0, M, N, K, stream) == 0
    torch.cuda.synchronize()
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.int8_mm_rescale(oracle.int_mm(a, w.T), rs, cs))
