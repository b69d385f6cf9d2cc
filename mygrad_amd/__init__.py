"""MI355X-native conv_nd / max_pool behind MyGrad's Operation contract.

    >>> import mygrad_amd as mg
    >>> from mygrad_amd.nnet import conv_nd, max_pool
    >>> out = max_pool(conv_nd(x, w, stride=1, padding=1), (2, 2), 2)
    >>> out.backward(g)        # x.grad, w.grad computed by the HIP kernels
    >>> loss = mg.sum(mg.nnet.relu(out) * g)   # relu, multiply and sum run on the device too

The arithmetic runs in ``libmygrad_hip.so`` (hand-written gfx950 kernels, called
through ctypes).  There is no CPU fallback: without the library or without a
gfx950 device the operations raise ``HipUnavailable``.
"""

from . import _device, _graph, _hip, nnet
from ._graph import mem_guard_off, mem_guard_on, no_autodiff
from ._hip import HipError, HipUnavailable, device_info, is_available, synchronize
from .errors import InvalidBackprop, InvalidGradient, SkipGradient
from .nnet.layers.utils import sliding_window_copy, sliding_window_view
from .operation_base import Operation
from .tensor_base import Tensor, asarray, device_tensor, tensor
from .math import matmul, multi_matmul, multiply, sum  # noqa: A004  (after tensor_base: the ops import Tensor)
from .tensor_manip import repeat
from .linalg import einsum
from . import linalg
from ._io import load, save

execute_op = Tensor._op

__all__ = [
    "Tensor",
    "tensor",
    "device_tensor",
    "asarray",
    "Operation",
    "execute_op",
    "no_autodiff",
    "mem_guard_off",
    "mem_guard_on",
    "sliding_window_view",
    "sliding_window_copy",
    "multiply",
    "einsum",
    "linalg",
    "matmul",
    "multi_matmul",
    "sum",
    "repeat",
    "save",
    "load",
    "nnet",
    "InvalidBackprop",
    "InvalidGradient",
    "SkipGradient",
    "HipError",
    "HipUnavailable",
    "device_info",
    "is_available",
    "synchronize",
]
