"""MI355X (gfx950) execution of the vpux hot path: ACT-SHAVE software kernels and the NCE/DPU
quantized convolution / matmul with the integer PPE, behind the C ABI in include/."""
from . import runtime  # noqa: F401

__all__ = ["runtime"]
