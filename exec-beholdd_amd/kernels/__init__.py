"""The gfx950 kernel library and its Python binding."""

from .library import HipKernels, KernelError
from . import build

__all__ = ["HipKernels", "KernelError", "build"]
