from .funcs import matmul

__all__ = ["matmul"]
