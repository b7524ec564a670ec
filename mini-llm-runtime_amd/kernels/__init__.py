from .build import BuildError, build_all, ensure_built, load
from .ops import Kernels, KernelError

__all__ = ["BuildError", "build_all", "ensure_built", "load", "Kernels", "KernelError"]
