import numpy as np

from ..tensor_base import Tensor
from .ops import EinSum

try:  # NumPy's own reading of the two calling conventions (what the reference uses as well)
    from numpy._core.einsumfunc import _parse_einsum_input
except ImportError:  # pragma: no cover
    from numpy.core.einsumfunc import _parse_einsum_input

__all__ = ["einsum"]


def _shape_only(tensor):
    """A stand-in with the tensor's shape and dtype that owns one element: NumPy's parser of the
    subscripts looks at the operands' shapes only, and a value that is on the device need not
    be copied to the host for that."""
    return np.broadcast_to(np.empty((), dtype=tensor.dtype), tensor.shape)


def einsum(*operands, optimize=False, out=None, constant=None):
    """einsum(subscripts, *operands)

    Einstein summation of the operands (reference: ``mygrad.einsum``,
    ``mygrad/linalg/funcs.py:178-451``), with back-propagation to each of them.

    Both of NumPy's calling conventions are read: ``einsum("ij,jk->ik", a, b)`` and
    ``einsum(a, [0, 1], b, [1, 2], [0, 2])``; without ``->`` the result holds the labels that
    occur once, in alphabetical order; ``...`` stands for the axes not named.

    Parameters
    ----------
    subscripts : str
        The labels of each operand's axes, separated by commas, and optionally those of
        the result after ``->``.
    operands : ArrayLike
        float32 / float64 operands.
    optimize : bool
        Accepted for compatibility; the order of evaluation is fixed.
    constant : Optional[bool]
        If True, the resulting Tensor is a constant.

    Returns
    -------
    Tensor

    Notes
    -----
    The summation runs on the matrix-product kernels after the operands have been transposed
    on the device.  More than two operands are contracted pairwise from the left; a label
    that occurs twice in one operand (``"ii"``: a trace or a diagonal) is taken along its
    diagonal first; an axis of length one is broadcast against a longer one under the
    same label.  ``out=`` takes a NumPy array, which receives the result and becomes the returned
    tensor's data (a tensor as the target asks for the reference's in-place graph semantics, which
    this package does not have: ``NotImplementedError``).  A tensor that occurs
    twice with the same labels receives one gradient, scaled by two, as in the reference.
    The result is a new array, where ``numpy.einsum`` may return a view.

    Examples
    --------
    >>> import mygrad_amd as mg
    >>> a = mg.Tensor([[0., 1.], [2., 3.], [4., 5.]])
    >>> b = mg.Tensor([[0., 1., 2.], [3., 4., 5.], [6., 7., 8.], [9., 10., 11.]])
    >>> mg.einsum("ki,jk->ij", a, b)
    Tensor([[10., 28., 46., 64.],
            [13., 40., 67., 94.]])
    """
    if isinstance(out, Tensor):
        raise NotImplementedError("einsum(..., out=<Tensor>) needs in-place operations on tensors, which are outside this package; pass an ndarray")
    operands = list(operands)
    if isinstance(operands[0], str):
        variables = operands[1:]
        operands[1:] = (_shape_only(var) if isinstance(var, Tensor) else var for var in operands[1:])
    else:
        end = -1 if len(operands) % 2 else None  # the last entry is the result's sublist
        variables = operands[:end:2]
        operands[:end:2] = (_shape_only(var) if isinstance(var, Tensor) else np.asarray(var) for var in operands[:end:2])
    in_lbls, out_lbls, _ = _parse_einsum_input(operands)
    return Tensor._op(
        EinSum,
        *variables,
        op_kwargs=dict(in_lbls=in_lbls, out_lbls=out_lbls, optimize=optimize, out=out),
        constant=constant,
    )
