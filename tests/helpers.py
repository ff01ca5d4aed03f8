"""Shared helpers for the test-suite (numpy <-> torch 16-bit float plumbing)."""
import numpy as np
import torch

TORCH_DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def bits_of(t: torch.Tensor) -> np.ndarray:
    """Storage of a CPU torch tensor as numpy: float32 stays, 16-bit floats become uint16."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float32:
        return t.numpy()
    return t.view(torch.int16).numpy().view(np.uint16)


def from_bits(a: np.ndarray, dtype: str) -> torch.Tensor:
    if dtype == "f32":
        return torch.from_numpy(np.ascontiguousarray(a, np.float32))
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(TORCH_DT[dtype])


def cast_bits(x32: np.ndarray, dtype: str) -> np.ndarray:
    """float32 numpy -> storage bits of `dtype`, rounded by torch (independent of the oracle)."""
    return bits_of(torch.from_numpy(np.ascontiguousarray(x32, np.float32)).to(TORCH_DT[dtype]))


def rel_err(a, b):
    """Normwise max error: max|a-b| / max|b|."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))
