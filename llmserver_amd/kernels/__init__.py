from . import build, library
from .library import KernelLibraryMissing
from .ops import HipOps, default_ops

__all__ = ["build", "library", "KernelLibraryMissing", "HipOps", "default_ops"]
