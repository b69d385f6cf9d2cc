from .funcs import matmul, multi_matmul

__all__ = ["matmul", "multi_matmul"]
