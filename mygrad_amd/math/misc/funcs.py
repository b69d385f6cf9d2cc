from ...tensor_base import Tensor
from .ops import MatMul

__all__ = ["matmul"]


def matmul(x1, x2, *, constant=None):
    """Matrix product of two tensors: ``matmul(x, y)`` is ``x @ y`` (reference:
    ``mygrad.matmul`` / ``numpy.matmul``).

    - If both arguments are 2-D they are multiplied like conventional matrices.
    - If either argument is N-D, N > 2, it is treated as a stack of matrices residing in
      the last two indexes.
    - A 1-D first argument is promoted to a matrix by prepending a 1 to its dimensions, a
      1-D second argument by appending a 1; the added dimension is removed afterwards.

    Multiplication by a scalar is not allowed (``ValueError``); two stacks must have the
    same batch shape (stacks that broadcast against each other are not part of this build).

    Parameters
    ----------
    x1, x2 : ArrayLike
        float32 or float64.
    constant : Optional[bool]
        If True, the resulting Tensor is a constant.

    Returns
    -------
    Tensor

    Examples
    --------
    >>> import mygrad_amd as mg
    >>> a = [[1., 0.], [0., 1.]]
    >>> b = [[4., 1.], [2., 2.]]
    >>> mg.matmul(a, b)
    Tensor([[4., 1.],
            [2., 2.]])
    >>> mg.matmul(a, [1., 2.])
    Tensor([1., 2.])
    """
    return Tensor._op(MatMul, x1, x2, constant=constant)
