"""Hand-written HIP kernels for gfx950, callable on torch tensors."""
from .hip_ops import HipOps, get_ops
from .library import KernelLibraryError, library_path, load_library

__all__ = ["HipOps", "get_ops", "KernelLibraryError", "library_path", "load_library"]
