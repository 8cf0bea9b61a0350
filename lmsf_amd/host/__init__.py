"""The engine's host runtime in C++ (cache manager, scheduler, step metadata), loaded through ctypes."""
from .library import HostLibraryError, load_host_library

__all__ = ["HostLibraryError", "load_host_library"]
