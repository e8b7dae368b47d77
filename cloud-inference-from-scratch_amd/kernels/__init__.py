from . import ops
from .library import KernelLibraryError, build_library, load_library

__all__ = ["KernelLibraryError", "build_library", "load_library", "ops"]
