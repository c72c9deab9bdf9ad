from . import kernels
from .library import KernelLibraryError, build, load_library

__all__ = ["KernelLibraryError", "build", "kernels", "load_library"]
