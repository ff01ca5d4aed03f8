import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _has_gpu():
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def kernel_override():
    """Pins a route for the duration of a test: kernel_override("int8_row", 1).  The library that ships has no such
    switch; the test-hook build of the same sources (libtpq_gfx950_hooks.so, tensorplay_amd/build.py) has, so for the
    test the operators are bound to that build."""
    import ctypes

    from tensorplay_amd import _lib, build

    assert os.path.exists(build.HOOKS_LIB_PATH), "build the test-hook library: python -m tensorplay_amd.build"
    _lib.load()  # torch's HIP runtime first, as for the shipped library
    shipped = _lib._lib
    hooked = _lib.bind(build.HOOKS_LIB_PATH)
    hooked.tpq_set_kernel_override.argtypes = [ctypes.c_char_p, ctypes.c_int]
    hooked.tpq_set_kernel_override.restype = ctypes.c_int
    _lib._lib = hooked
    touched = []

    def pin(route: str, value: int) -> None:
        assert hooked.tpq_set_kernel_override(route.encode(), value) == 0, _lib.last_error()
        touched.append(route)

    try:
        yield pin
    finally:
        for route in touched:
            hooked.tpq_set_kernel_override(route.encode(), -1)
        _lib._lib = shipped
