from . import build, ops
from .ops import KernelRefused

__all__ = ["build", "ops", "KernelRefused"]
