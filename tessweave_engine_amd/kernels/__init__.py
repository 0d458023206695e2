"""Hand-written HIP kernels for gfx950: build, ctypes binding, checked wrappers."""
from . import build, lib, ops
from .lib import KernelError

__all__ = ["build", "lib", "ops", "KernelError"]
