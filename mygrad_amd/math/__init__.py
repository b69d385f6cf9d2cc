"""Element-wise and sequential operations that sit either side of ``conv_nd`` /
``max_pool`` in a chain and run on the device: ``multiply`` and ``sum``."""

from .arithmetic.funcs import multiply
from .sequential.funcs import sum  # noqa: A004 (same name as the reference's mygrad.sum)

__all__ = ["multiply", "sum"]
