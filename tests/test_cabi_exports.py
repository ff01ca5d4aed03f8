"""The C-ABI library loads without a GPU and exports every symbol include/tpq.h declares."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "tpq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tpq_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared()
    for must in ("tpq_quantize_rowwise", "tpq_int_mm", "tpq_int8_mm_rescale", "tpq_int8_mm_dequant", "tpq_int4_pack",
                 "tpq_int4_mm", "tpq_ternary_pack", "tpq_ternary_unpack", "tpq_ternary_mm", "tpq_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from tensorplay_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} not built: run `python -m tensorplay_amd.build`")
    lib = _lib.load()
    for name in _declared():
        assert hasattr(lib, name), f"{name} declared in include/tpq.h but not exported"
    assert set(_lib.SIGNATURES) | {"tpq_last_error"} == set(_declared())
    assert lib.tpq_abi_version() == 1
    assert isinstance(_lib.last_error(), str)


def test_argument_validation_needs_no_gpu():
    """Shape/type checks run on the host before any launch."""
    from tensorplay_amd import _lib

    lib = _lib.load()
    assert lib.tpq_int4_pack(None, 8, 33, 2, None, None) == _lib.TPQ_ERR_INVALID_VALUE
    assert "K must be even" in _lib.last_error()
    assert lib.tpq_int4_pack(None, 8, 32, 3, None, None) == _lib.TPQ_ERR_INVALID_VALUE
    assert lib.tpq_quantize_rowwise(None, 7, 1, 1, 1e-5, 127.0, -127, 127, 0, None, None, None) == _lib.TPQ_ERR_INVALID_TYPE
    assert lib.tpq_int4_mm(None, 1, 1, 64, None, 2, 8, 48, None, None, None) == _lib.TPQ_ERR_INVALID_VALUE
    assert lib.tpq_int4_mm(None, 1, 1, 64, None, 4, 8, 32, None, None, None) == _lib.TPQ_ERR_UNSUPPORTED
    # zero-sized problems succeed without touching the device
    assert lib.tpq_quantize_rowwise(None, 0, 0, 16, 1e-5, 127.0, -127, 127, 0, None, None, None) == _lib.TPQ_OK
    assert lib.tpq_int_mm(None, 0, None, 1, 1, None, 0, 4, 4, None) == _lib.TPQ_OK
    assert lib.tpq_ternary_mm(None, None, None, 1.0, None, 0, 4, 4, None, 0, None, None) == _lib.TPQ_OK


def test_int8_workspace_sizing_is_host_logic():
    """tpq_int8_mm_workspace_bytes: slices x M x N x 4 bytes where the k range is cut, 0 where one launch does it."""
    from tensorplay_amd import _lib

    lib = _lib.load()
    ws = lib.tpq_int8_mm_workspace_bytes
    assert ws(16, 4096, 4096) == 0            # decode kernel
    assert ws(32, 4096, 4096) == 0
    assert ws(2048, 4096, 4096) == 0          # 256 tiles fill the chip
    assert ws(128, 4096, 4096) == 8 * 128 * 4096 * 4     # 32 tiles of 256 x 128 -> 8 slices of 4 stages
    assert ws(512, 4096, 4096) == 0           # one round of 128 x 128 tiles is estimated faster than 4 slices + the adding pass
    assert ws(256, 4096, 11008) == 8 * 256 * 4096 * 4    # few tiles, long K: 32 tiles of 256 x 128 -> 8 slices
    assert ws(128, 8192, 8192) == 4 * 128 * 8192 * 4     # 64 tiles -> 4 slices of 16 stages
    assert ws(128, 4096, 512) == 0            # K of four stages: nothing to cut
    assert ws(128, 4096, 4100) == 0           # K not a multiple of the stage
    assert ws(0, 4096, 4096) == 0 and ws(128, 0, 4096) == 0
    # a NULL workspace is the plain entry point: same argument checks, no launch for empty problems
    assert lib.tpq_int8_mm_dequant_ws(None, None, None, None, None, None, 0, 0, 8, 8, None, 0, None) == _lib.TPQ_OK
    assert lib.tpq_int8_mm_dequant_ws(None, None, None, None, None, None, 7, 4, 8, 8, None, 0, None) == _lib.TPQ_ERR_INVALID_TYPE
    assert lib.tpq_int_mm_ws(None, 0, None, 1, 1, None, 0, 4, 4, None, 0, None) == _lib.TPQ_OK


def test_int4_rows_workspace_sizing_is_host_logic():
    """tpq_int4_mm_rows_workspace_bytes: the decode kernels' share, and for 33 .. 256 rows the fp32 sums of the slices
    the tiled kernel would take (counters + slices x M x N x 4)."""
    from tensorplay_amd import _lib

    lib = _lib.load()
    base, rows = lib.tpq_int4_mm_workspace_bytes, lib.tpq_int4_mm_rows_workspace_bytes
    counters = 4096 * 4
    assert rows(1, 11008, 4096) == base(11008) and rows(32, 4096, 4096) == base(4096)
    assert rows(128, 4096, 4096) == counters + 4 * 128 * 4096 * 4      # 64 workgroups of 64 channels -> four slices
    assert rows(255, 4096, 4096) == counters + 2 * 255 * 4096 * 4      # 128 workgroups -> two
    assert rows(128, 4096, 11008) == counters + 4 * 128 * 4096 * 4     # long K, few channels
    assert rows(128, 11008, 4096) == base(11008)                       # 172 workgroups: one slice, nothing to add up
    assert rows(300, 4096, 4096) == base(4096)                         # beyond 256 rows: no slices
    assert rows(128, 4096, 512) == base(4096)                          # K of four steps: nothing to cut
    assert rows(0, 4096, 4096) == base(4096) and rows(128, 0, 4096) == 0


def test_bench_refuses_more_than_one_gpu():
    """The benchmark is a one-GPU program: any other --gpus value exits with a message and status 2."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    run = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert run.returncode == 2 and "ONE GPU" in run.stderr


def test_dispatch_does_not_depend_on_the_environment():
    """The shipped library imports no getenv and exports neither the route switch of the test-hook build nor the
    measurement probe: which kernel runs is a function of the arguments, and the interface lists operators only."""
    import ctypes
    import subprocess
    from tensorplay_amd import _lib, build

    _lib.load()
    syms = subprocess.run(["nm", "-D", "--undefined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    assert "getenv" not in syms, "the library was built with -DTPQ_TUNING (sweep knobs compiled in)"
    exported = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    assert "tpq_set_kernel_override" not in exported and "tpq_probe_read" not in exported
    assert "tpq_quantize_stamps_read" not in exported and "g_quant_stamps" not in exported   # clock readings: the measuring build only
    # the test-hook build validates its arguments on the host
    hooked = ctypes.CDLL(build.HOOKS_LIB_PATH)
    hooked.tpq_set_kernel_override.argtypes = [ctypes.c_char_p, ctypes.c_int]
    hooked.tpq_last_error.restype = ctypes.c_char_p
    assert hooked.tpq_set_kernel_override(b"int8_row", 1) == 0 and hooked.tpq_set_kernel_override(b"int8_row", -1) == 0
    assert hooked.tpq_set_kernel_override(b"lowbit_row", 0) == 0 and hooked.tpq_set_kernel_override(b"lowbit_row", -1) == 0
    assert hooked.tpq_set_kernel_override(b"int4_row", 1) == 0 and hooked.tpq_set_kernel_override(b"int4_row", -1) == 0
    assert hooked.tpq_set_kernel_override(b"no_such_route", 1) == _lib.TPQ_ERR_INVALID_VALUE
    assert b"unknown route" in hooked.tpq_last_error()
    assert hooked.tpq_set_kernel_override(b"int8_row", 5) == _lib.TPQ_ERR_INVALID_VALUE
    assert hooked.tpq_set_kernel_override(None, 0) == _lib.TPQ_ERR_INVALID_VALUE
    # the measuring build of the row quantizer: the operator plus the reader of its clock readings, argument checks on the host
    stamps = ctypes.CDLL(build.QUANT_STAMPS_LIB_PATH)
    stamps.tpq_quantize_stamps_read.argtypes = [ctypes.c_void_p, ctypes.c_int64]
    assert stamps.tpq_quantize_stamps_read(None, 8) == _lib.TPQ_ERR_INVALID_VALUE
    assert stamps.tpq_quantize_stamps_read(16, 1 << 20) == _lib.TPQ_ERR_INVALID_VALUE
    assert hasattr(stamps, "tpq_quantize_rowwise")
    # the probe library: argument checks of the column pattern, no launch
    probe = ctypes.CDLL(build.PROBE_LIB_PATH)
    probe.tpq_probe_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    assert probe.tpq_probe_read(16, 1024, 1, 8, 8, 32, 16, None) == _lib.TPQ_ERR_INVALID_VALUE   # fewer bytes than one tile row
    assert probe.tpq_probe_read(16, 1 << 30, 1, 8, 8, 5000, 16, None) == _lib.TPQ_ERR_INVALID_VALUE
    assert probe.tpq_probe_read(16, 16384 * 8, 1, 8, 7, 32, 16, None) == _lib.TPQ_ERR_INVALID_VALUE
