"""Element-wise, sequential and matrix operations that sit either side of ``conv_nd`` /
``max_pool`` in a chain and run on the device: ``multiply``, ``sum`` and ``matmul``."""

from .arithmetic.funcs import multiply
from .misc.funcs import matmul, multi_matmul
from .sequential.funcs import sum  # noqa: A004 (same name as the reference's mygrad.sum)

__all__ = ["multiply", "matmul", "multi_matmul", "sum"]
