"""Hand-written HIP kernels for gfx950 and their Python faces."""

from . import ops
from .ops import KernelError

__all__ = ["KernelError", "ops"]
