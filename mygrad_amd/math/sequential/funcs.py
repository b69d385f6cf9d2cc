from ...tensor_base import Tensor
from .ops import Sum

__all__ = ["sum"]


def sum(x, axis=None, keepdims=False, *, constant=None):  # noqa: A001
    """Sum of all tensor elements (reference: ``mygrad.sum``).

    Parameters
    ----------
    x : ArrayLike
        float32 or float64.
    axis : None
        Only the full reduction runs on the GPU; anything else raises
        ``NotImplementedError``.
    keepdims : bool
        Keep the reduced axes with length one.
    constant : Optional[bool]
        If True, the resulting Tensor is a constant.

    Returns
    -------
    Tensor

    Examples
    --------
    >>> import mygrad_amd as mg
    >>> x = mg.Tensor([1.0, 2.0, 3.0])
    >>> mg.sum(x).backward()
    >>> x.grad
    array([1., 1., 1.])
    """
    return Tensor._op(Sum, x, op_args=(axis, keepdims), constant=constant)
