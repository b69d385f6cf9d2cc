from .funcs import sum  # noqa: A004
from .ops import Sum

__all__ = ["sum", "Sum"]
