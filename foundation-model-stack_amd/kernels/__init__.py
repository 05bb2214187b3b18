from . import ops
from .build import build, ensure_built
from .library import KernelError, KernelLibraryMissing, load

__all__ = ["ops", "build", "ensure_built", "load", "KernelError", "KernelLibraryMissing"]
