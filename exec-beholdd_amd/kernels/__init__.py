"""The gfx950 kernel library and its Python binding."""

from .library import HipKernels, KernelError, KernelSizes, NormedRows, PackedWeight, PartSums
from . import build

__all__ = ["HipKernels", "KernelError", "KernelSizes", "NormedRows", "PackedWeight", "PartSums", "build"]
