"""Hand-written gfx950 kernels and their tensor-level wrappers."""
from . import ops
from .library import KernelError, check_device, library_path, load

__all__ = ["ops", "KernelError", "check_device", "library_path", "load"]
