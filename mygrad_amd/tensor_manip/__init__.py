"""Tensor-manipulation operations that run on the device: ``repeat``."""

from .tiling.funcs import repeat

__all__ = ["repeat"]
