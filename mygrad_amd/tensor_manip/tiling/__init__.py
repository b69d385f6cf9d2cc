from .funcs import repeat

__all__ = ["repeat"]
