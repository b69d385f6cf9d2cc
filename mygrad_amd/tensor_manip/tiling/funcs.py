"""``repeat``: the user-facing function over the ``Repeat`` operation (reference:
``mygrad/tensor_manip/tiling/funcs.py``, itself modelled on ``numpy.repeat``)."""

from ...tensor_base import Tensor
from .ops import Repeat

__all__ = ["repeat"]


def repeat(a, repeats, axis=None, *, constant=None):
    """Copy every entry of ``a`` along ``axis`` a given number of times, on the GPU.

    ``repeats`` is one count for all entries or one count per entry of the axis (zeros
    allowed); with ``axis=None`` the input is read as flattened and the result is 1-D, as
    with ``numpy.repeat``.  Any dtype of 1, 2, 4 or 8 bytes is accepted (integer tensors come
    back constant); the gradient -- each input entry collects the gradient of its copies --
    is defined for float32 / float64.

    >>> import mygrad_amd as mg
    >>> x = mg.Tensor([[1., 2.], [3., 4.]])
    >>> y = mg.repeat(x, [1, 2], axis=0)
    >>> y.data
    array([[1., 2.],
           [3., 4.],
           [3., 4.]])
    >>> y.backward()
    >>> x.grad
    array([[1., 1.],
           [2., 2.]])
    """
    return Tensor._op(Repeat, a, op_args=(repeats, axis), constant=constant)
