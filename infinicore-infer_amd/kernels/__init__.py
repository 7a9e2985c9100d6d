"""ctypes bindings of the HIP kernels under csrc/ (built for gfx950)."""
from .lib import KernelError, get_lib, library_path
from . import ops

__all__ = ["KernelError", "get_lib", "library_path", "ops"]
