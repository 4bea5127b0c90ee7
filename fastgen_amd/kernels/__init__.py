"""Hand-written HIP kernels for gfx950 and their Python faces."""
from . import ops
from ._lib import KernelBuildError, build_all
from .ops import KernelArgumentError

__all__ = ["ops", "build_all", "KernelBuildError", "KernelArgumentError"]
