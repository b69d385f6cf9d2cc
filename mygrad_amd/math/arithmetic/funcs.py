from ...tensor_base import Tensor
from .ops import Multiply

__all__ = ["multiply"]


def multiply(x1, x2, *, constant=None):
    """Multiply the arguments element-wise (reference: ``mygrad.multiply``).

    Parameters
    ----------
    x1, x2 : ArrayLike
        float32 or float64 operands that broadcast against each other.
    constant : Optional[bool]
        If True, the resulting Tensor is a constant.

    Returns
    -------
    Tensor

    Examples
    --------
    >>> import mygrad_amd as mg
    >>> x = mg.Tensor([1.0, 2.0, 3.0])
    >>> y = mg.multiply(x, [2.0, 2.0, 2.0])
    >>> y.backward()
    >>> x.grad
    array([2., 2., 2.])
    >>> scale = mg.Tensor([10.0, 100.0])
    >>> mg.multiply(mg.Tensor([[1.0, 2.0], [3.0, 4.0]]), scale).backward()
    >>> scale.grad   # summed over the axis it was broadcast along
    array([4., 6.])
    """
    return Tensor._op(Multiply, x1, x2, constant=constant)
