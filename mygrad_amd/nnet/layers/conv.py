"""``conv_nd`` on the MI355X: the ConvND operation with the reference's
signature, argument checks and errors (``mygrad/nnet/layers/conv.py``), whose
forward pass, ``dx`` and ``dw`` run as implicit-GEMM kernels in
``libmygrad_hip.so``."""

from numbers import Integral

import numpy as np

from ... import _device, _hip
from . import _highrank
from ...operation_base import Operation
from ...tensor_base import Tensor
from .utils import check_window_args

__all__ = ["conv_nd", "ConvND"]


def _per_axis(value, m, lowest):
    """int-or-sequence -> length-m int array, with the reference's assertion
    (conv.py:35-61): right length, every entry an integer >= ``lowest``."""
    arr = np.array((value,) * m) if isinstance(value, Integral) else np.array(value, dtype=int)
    assert len(arr) == m and all(v >= lowest and isinstance(v, Integral) for v in arr)
    return arr


def _kernel_dtype(*arrays):
    """The dtype the kernels compute in: NumPy's promotion of the operands, which
    must come out as float32 or float64."""
    dtype = np.result_type(*(a.dtype for a in arrays))
    if dtype not in (np.float32, np.float64):
        raise TypeError(
            f"conv_nd runs on the GPU in float32 or float64; the operands promote to {dtype} "
            "(there is no CPU fallback)"
        )
    return np.dtype(dtype)


def _device_zeros(shape, dtype):
    """Zero-filled result of an empty problem, produced on the device like any other."""
    count = int(np.prod(shape, dtype=np.int64))
    buf = _device.DeviceBuffer(count * dtype.itemsize)
    _hip.check(_hip.lib().mg_memset_zero(buf.ptr, count * dtype.itemsize))
    return _device.download(buf, shape, dtype)


class ConvND(Operation):
    """N-dimensional strided, dilated, zero-padded cross-correlation.

    ``(N, C, X0, ...) * (F, C, W0, ...) -> (N, F, G0, ...)``
    """

    takes_device_arrays = True

    gradient_on_device = True

    def __call__(self, x, w, *, stride, padding=0, dilation=1):
        self.variables = (x, w)
        xd, wd = _device.value_of(x), _device.value_of(w)

        assert xd.ndim > 2
        assert xd.ndim == wd.ndim
        assert wd.shape[1] == xd.shape[1], "The channel-depth of the batch and filters must agree"

        m = wd.ndim - 2
        x_shape = np.array(xd.shape[2:])
        w_shape = np.array(wd.shape[2:])
        dilation = _per_axis(dilation, m, 1)
        padding = _per_axis(padding, m, 0)
        stride = _per_axis(stride, m, 1)

        out_shape = (x_shape + 2 * padding - ((w_shape - 1) * dilation + 1)) / stride + 1
        if not all(i.is_integer() and i > 0 for i in out_shape):
            raise ValueError(
                "Stride and kernel dimensions are incompatible: \n"
                f"Input dimensions: {tuple(x_shape)}\n"
                f"Stride dimensions: {tuple(stride)}\n"
                f"Kernel dimensions: {tuple(w_shape)}\n"
                f"Padding dimensions: {tuple(padding)}\n"
                f"Dilation dimensions: {tuple(dilation)}\n"
            )
        self.padding, self.stride, self.dilation = padding, stride, dilation

        # the window helper's own checks, applied to the padded extent (the
        # reference windows the padded array: conv.py:81-88)
        padded = tuple(xd.shape[:2]) + tuple(int(n + 2 * p) for n, p in zip(x_shape, padding))
        check_window_args(padded, tuple(int(i) for i in w_shape), tuple(int(s) for s in stride),
                          tuple(int(d) for d in dilation))

        dtype = _kernel_dtype(xd, wd)
        grid = tuple(int(g) for g in out_shape)
        out_full = (xd.shape[0], wd.shape[0], *grid)
        self._dtype = dtype
        self._grid = grid
        if xd.size == 0 or wd.size == 0:
            # nothing to gather: every product involves a padding zero
            self._desc = None
            return _device_zeros(out_full, dtype)

        xb = _device.to_device(xd, dtype)
        wb = _device.to_device(wd, dtype)
        if m > _hip.MG_MAX_ND:
            # more convolved axes than the kernels take: the leading ones are taken apart on the
            # host, tap by tap, into convolutions over the last three (same results, more launches)
            self._desc = "folded"
            ob = _highrank.conv_forward(xb, wb, dtype, tuple(xd.shape), tuple(wd.shape), grid, stride, padding, dilation)
        else:
            self._desc = _hip.conv_desc(dtype, xd.shape, wd.shape, grid, stride, padding, dilation)
            ob = _device.DeviceBuffer(int(np.prod(out_full)) * dtype.itemsize)
            _hip.check(_hip.lib().mg_conv_fwd(self._desc, xb.ptr, wb.ptr, ob.ptr))
        out = _device.download(ob, out_full, dtype)
        _device.attach(out, ob)
        return out

    def backward_var(self, grad, index, **kwargs):
        x, w = (_device.value_of(v) for v in self.variables)
        dtype = self._dtype
        if self._desc is None:
            return _device_zeros((x if index == 0 else w).shape, dtype)
        lib = _hip.lib()
        if tuple(grad.shape) != (x.shape[0], w.shape[0], *self._grid):
            raise ValueError(f"conv_nd backward: gradient of shape {tuple(grad.shape)} for an output of shape "
                             f"{(x.shape[0], w.shape[0], *self._grid)}")
        gb = _device.to_device(grad, dtype)
        folded = (dtype, tuple(x.shape), tuple(w.shape), self._grid, self.stride, self.padding, self.dilation)
        if index == 0:  # dx
            wb = _device.to_device(w, dtype)
            if self._desc == "folded":
                db = _highrank.conv_dgrad(gb, wb, *folded)
            else:
                db = _device.DeviceBuffer(x.size * dtype.itemsize)
                _hip.check(lib.mg_conv_dgrad(self._desc, gb.ptr, wb.ptr, db.ptr))
            out = _device.download(db, x.shape, dtype)
        else:  # dw
            xb = _device.to_device(x, dtype)
            if self._desc == "folded":
                db = _highrank.conv_wgrad(gb, xb, *folded)
            else:
                db = _device.DeviceBuffer(w.size * dtype.itemsize)
                _hip.check(lib.mg_conv_wgrad(self._desc, gb.ptr, xb.ptr, db.ptr))
            out = _device.download(db, w.shape, dtype)
        _device.attach_transient(out, db)
        return out


def conv_nd(x, filter_bank, *, stride, padding=0, dilation=1, constant=None):
    """Use ``filter_bank`` (``w``) to perform strided N-dimensional neural
    network-style convolutions over ``x``::

        f(x, w) -> x * w        (N, C, X0, ...) * (F, C, W0, ...) -> (N, F, G0, ...)

    The filters are not flipped (a cross-correlation), and only 'valid'
    placements of the filters over the zero-padded data are used.

    Parameters
    ----------
    x : ArrayLike, shape=(N, C, X0, ...)
        The data batch to be convolved over.
    filter_bank : ArrayLike, shape=(F, C, W0, ...)
        The filters used to perform the convolutions.
    stride : Union[int, Tuple[int, ...]]
        (keyword-only) Step size of the filter placements along each convolved axis.
    padding : Union[int, Tuple[int, ...]]
        (keyword-only) Number of zeros padded to both ends of each convolved axis.
    dilation : Union[int, Tuple[int, ...]], optional (default=1)
        (keyword-only) Spacing between filter elements along each convolved axis:
        placement ``i`` multiplies the filter against ``x[:, :, i*s : i*s + w*d : d]``.
    constant : Optional[bool]
        If True, the resulting Tensor is a constant.

    Returns
    -------
    Tensor, shape=(N, F, G0, ...)

    Raises
    ------
    ValueError
        ``x`` has fewer than three dimensions, ``x`` and ``filter_bank`` differ in
        dimensionality or channel depth, or ``(X + 2p - ((W-1)d + 1)) / s + 1`` is
        not a positive integer along some axis.
    AssertionError
        ``stride`` / ``padding`` / ``dilation`` has the wrong length or a bad value.

    Examples
    --------
    >>> import numpy as np
    >>> from mygrad_amd import Tensor
    >>> from mygrad_amd.nnet import conv_nd
    >>> x = np.zeros((1, 1, 16)); x[..., 5:11] = 1      # a square wave
    >>> x = Tensor(x); k = Tensor(np.ones((1, 1, 5)))    # a box kernel
    >>> out = conv_nd(x, k, stride=1)                    # triangle response
    >>> out.backward()
    >>> k.grad
    array([[[6., 6., 6., 6., 6.]]])
    """
    if x.ndim < 3:
        raise ValueError(f"`x` must possess at least three dimensions, got {x.ndim} dimensions")
    if x.ndim != filter_bank.ndim:
        raise ValueError(
            f"`x` ({x.ndim}-dimensions) must have the same dimensionality as "
            f"`filter_bank` ({filter_bank.ndim}-dimensions)"
        )
    if filter_bank.shape[1] != x.shape[1]:
        raise ValueError(
            f"`x.shape[1]` ({x.shape[1]}) must match `filter_bank.shape[1]` ({filter_bank.shape[1]})"
        )
    return Tensor._op(
        ConvND,
        x,
        filter_bank,
        op_kwargs={"stride": stride, "padding": padding, "dilation": dilation},
        constant=constant,
    )
