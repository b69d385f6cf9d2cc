from .relu import relu

__all__ = ["relu"]
