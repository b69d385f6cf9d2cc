from .batchnorm import batchnorm
from .conv import conv_nd
from .pooling import max_pool
from .utils import sliding_window_copy, sliding_window_view

__all__ = ["batchnorm", "conv_nd", "max_pool", "sliding_window_copy", "sliding_window_view"]
