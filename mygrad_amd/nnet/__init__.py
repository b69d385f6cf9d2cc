from .activations import relu
from .layers import conv_nd, max_pool

__all__ = ["conv_nd", "max_pool", "relu"]
