"""Einstein summation on the device (reference: ``mygrad/linalg``)."""

from .funcs import einsum
from .ops import EinSum

__all__ = ["einsum", "EinSum"]
