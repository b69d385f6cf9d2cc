from ...tensor_base import Tensor
from .ops import MatMul

__all__ = ["matmul", "multi_matmul"]


def matmul(x1, x2, *, constant=None):
    """Matrix product of two tensors: ``matmul(x, y)`` is ``x @ y`` (reference:
    ``mygrad.matmul`` / ``numpy.matmul``).

    - If both arguments are 2-D they are multiplied like conventional matrices.
    - If either argument is N-D, N > 2, it is treated as a stack of matrices residing in
      the last two indexes.
    - A 1-D first argument is promoted to a matrix by prepending a 1 to its dimensions, a
      1-D second argument by appending a 1; the added dimension is removed afterwards.

    Multiplication by a scalar is not allowed (``ValueError``); two stacks broadcast against
    each other like NumPy's.

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


def _chain_split(dims):
    """Where to cut each run of a matrix chain so that the number of scalar multiplications is
    smallest: ``dims[i], dims[i + 1]`` are the rows and columns of matrix ``i``.  Returns
    ``cut`` with ``cut[i][j]`` = index of the last matrix of the left part of the run
    ``i..j`` (the textbook dynamic programme over run lengths)."""
    n = len(dims) - 1
    cost = [[0.0] * n for _ in range(n)]
    cut = [[0] * n for _ in range(n)]
    for length in range(2, n + 1):
        for i in range(n - length + 1):
            j = i + length - 1
            best = None
            for k in range(i, j):
                c = cost[i][k] + cost[k + 1][j] + float(dims[i]) * dims[k + 1] * dims[j + 1]
                if best is None or c < best:
                    best, cut[i][j] = c, k
            cost[i][j] = best
    return cut


def multi_matmul(tensors, *, constant=None):
    """Matrix product of two or more tensors, multiplied in the order that needs the fewest
    scalar multiplications (reference: ``mygrad.multi_matmul``,
    ``mygrad/math/misc/funcs.py:638-851``).

    Parameters
    ----------
    tensors : Sequence[ArrayLike]
        One- or two-dimensional, float32 or float64.  A one-dimensional first operand is a row
        vector, a one-dimensional last operand a column vector; the operands in between
        must be two-dimensional.
    constant : Optional[bool]
        If True, the resulting Tensor is a constant.

    Returns
    -------
    Tensor
        ``tensors[0] @ tensors[1] @ ...``: a matrix, a vector if the first or the last
        operand is one-dimensional, a scalar if both are.

    Raises
    ------
    ValueError
        Fewer than two operands, or an operand that is not one- or two-dimensional.

    Examples
    --------
    >>> import numpy as np
    >>> import mygrad_amd as mg
    >>> a, b, c = mg.Tensor(np.ones((10, 100))), mg.Tensor(np.ones((100, 5))), mg.Tensor(np.ones((5, 50)))
    >>> mg.multi_matmul([a, b, c]).shape   # computed as (a @ b) @ c: 7500 multiplications, not 75000
    (10, 50)
    """
    tensors = [t if isinstance(t, Tensor) else Tensor(t, constant=True, copy=False) for t in tensors]
    for t in tensors:
        if not 1 <= t.ndim <= 2:
            raise ValueError(f"{t.ndim}-dimensional tensor given. Tensor must be one or two-dimensional")
    n = len(tensors)
    if n < 2:
        raise ValueError("Expecting at least two arrays.")
    if n == 2:
        return matmul(tensors[0], tensors[1], constant=constant)
    for t in tensors[1:-1]:
        if t.ndim != 2:
            raise ValueError("the operands between the first and the last must be two-dimensional")
    # rows of every operand, then the columns of the last: a vector counts as one row / one column
    dims = [t.shape[0] if t.ndim == 2 else 1 for t in tensors[:-1]]
    dims += [tensors[-1].shape[0], tensors[-1].shape[1] if tensors[-1].ndim == 2 else 1]
    cut = _chain_split(dims)

    def product(i, j):
        if i == j:
            return tensors[i]
        k = cut[i][j]
        return matmul(product(i, k), product(k + 1, j), constant=constant)

    return product(0, n - 1)
