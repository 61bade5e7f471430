from .library import KernelError
from .ops import HipKernels

__all__ = ["KernelError", "HipKernels"]
