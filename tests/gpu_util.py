"""Helpers for the GPU parity tests: numpy <-> device tensors, oracle dtype tags."""
import numpy as np
import torch

from helpers import TORCH_DT, bits_of, cast_bits, from_bits, rel_err  # noqa: F401

DEV = "cuda:0"


def dev(a: np.ndarray, dtype: str = None) -> torch.Tensor:
    """numpy array (or 16-bit float bit pattern with its dtype tag) -> device tensor."""
    if dtype in ("f16", "bf16"):
        return from_bits(a, dtype).to(DEV)
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t: torch.Tensor) -> np.ndarray:
    """device tensor -> numpy (16-bit floats come back as uint16 bit patterns)."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.float16, torch.bfloat16):
        return bits_of(t)
    return t.numpy()


def assert_close_norm(got, want, tol, what=""):
    """Normwise bound max|got-want| <= tol * max|want| plus the elementwise bound
    |got-want| <= tol * (rms(want) + |want|)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    err = np.abs(got - want)
    scale = max(np.abs(want).max(), 1e-30)
    assert err.max() <= tol * scale, f"{what}: normwise error {err.max() / scale:.3e} > {tol:.1e}"
    rms = np.sqrt(np.mean(want ** 2))
    bad = err > tol * (rms + np.abs(want))
    assert not bad.any(), f"{what}: {bad.sum()} elements outside |d| <= {tol:.0e} (rms + |ref|)"
