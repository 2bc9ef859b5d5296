from . import kernels, library
from .library import KernelLibraryError

__all__ = ["kernels", "library", "KernelLibraryError"]
