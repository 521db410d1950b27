from . import kernels
from .library import KernelLibraryError, library

__all__ = ["kernels", "library", "KernelLibraryError"]
