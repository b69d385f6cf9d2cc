from .funcs import multiply
from .ops import Multiply

__all__ = ["multiply", "Multiply"]
