"""Host-side counterpart of the reference's ``tensorplay.ao`` for the quantized-linear path."""
from . import quantization  # noqa: F401
