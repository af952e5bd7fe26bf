"""The HIP kernels: building and loading them (``library``) and calling them on tensors (``ops``)."""
from .library import KernelBuildError, KernelError

__all__ = ["KernelBuildError", "KernelError"]
