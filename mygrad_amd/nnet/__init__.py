from .activations import relu
from .layers import batchnorm, conv_nd, max_pool

__all__ = ["batchnorm", "conv_nd", "max_pool", "relu"]
