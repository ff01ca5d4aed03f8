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
    """Pins one of the library's two selectable routes for the duration of a test: kernel_override("int8_row", 1)."""
    from tensorplay_amd import _lib

    lib = _lib.load()
    touched = []

    def pin(route: str, value: int) -> None:
        assert lib.tpq_set_kernel_override(route.encode(), value) == 0, _lib.last_error()
        touched.append(route)

    yield pin
    for route in touched:
        lib.tpq_set_kernel_override(route.encode(), -1)
