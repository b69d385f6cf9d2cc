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


_PLAIN = (int, tuple)  # settings that hash: the usual way to pass stride, padding and dilation
_CHECKED = {}          # (x.shape, w.shape, stride, padding, dilation) -> what ConvND.__call__ derives from them


def _per_axis(value, m, lowest):
    """int-or-sequence -> length-m int array, with the reference's assertion
    (conv.py:35-61): right length, every entry an integer >= ``lowest``."""
    arr = np.array((value,) * m) if isinstance(value, Integral) else np.array(value, dtype=int)
    assert len(arr) == m and all(v >= lowest and isinstance(v, Integral) for v in arr)
    return arr


def _kernel_dtype(*arrays):
    """(the dtype the kernels compute in, the dtype of the result): NumPy's promotion of the
    operands, which must come out as float32, float64 or float16.  float16 is a storage type:
    NumPy multiplies float16 arrays with float32 sums rounded once at the end
    (``np.tensordot`` in the reference's conv.py:96-99), so its operands are widened to float32
    (exactly), the float32 kernels run, and the result is rounded to float16 on the device."""
    dtype = np.dtype(np.result_type(*(a.dtype for a in arrays)))
    if dtype == np.float16:
        return np.dtype(np.float32), dtype
    if dtype.kind in "iu":
        # Integer operands (constants: the reference multiplies them with np.tensordot in integer
        # arithmetic, conv.py:96-99).  float64 holds every integer below 2**53, so while no sum of
        # products can reach that, the float64 kernels give the integer result exactly.
        return np.dtype(np.float64), dtype
    if dtype not in (np.float32, np.float64):
        raise TypeError(
            f"conv_nd runs on the GPU in float32 or float64 (float16 operands are widened to float32); "
            f"the operands promote to {dtype} (there is no CPU fallback)"
        )
    return dtype, dtype


def _narrowed(buf, shape, dtype, result_dtype):
    """The kernel's result ``buf`` as the array handed back: rounded to float16 on the device
    when the operands were float16."""
    if result_dtype != dtype:
        buf = _device.DeviceArray(buf, shape, dtype).astype(result_dtype).buf
    return _device.download(buf, shape, result_dtype), buf


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
        # A layer is called with the same shapes and settings at every step: what the checks below
        # made of them the first time (they passed) is kept and handed out again.
        key = None
        if type(stride) in _PLAIN and type(padding) in _PLAIN and type(dilation) in _PLAIN:
            key = (tuple(xd.shape), tuple(wd.shape), stride, padding, dilation)
        try:
            checked = _CHECKED.get(key) if key is not None else None
        except TypeError:  # a tuple of something that does not hash
            key = checked = None
        if checked is None:
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

            # the window helper's own checks, applied to the padded extent (the
            # reference windows the padded array: conv.py:81-88)
            padded = tuple(xd.shape[:2]) + tuple(int(n + 2 * p) for n, p in zip(x_shape, padding))
            check_window_args(padded, tuple(int(i) for i in w_shape), tuple(int(s) for s in stride),
                              tuple(int(d) for d in dilation))
            for arr in (padding, stride, dilation):
                arr.flags.writeable = False  # shared between the operations that hit this entry
            checked = (padding, stride, dilation, tuple(int(g) for g in out_shape))
            if key is not None:
                if len(_CHECKED) >= 1024:
                    _CHECKED.clear()
                _CHECKED[key] = checked
        padding, stride, dilation, out_shape = checked
        self.padding, self.stride, self.dilation = padding, stride, dilation

        if np.iscomplexobj(xd) or np.iscomplexobj(wd):
            return self._complex_forward(xd, wd)
        dtype, result_dtype = _kernel_dtype(xd, wd)
        if result_dtype.kind in "iu" and xd.size and wd.size:
            xd, wd = np.asarray(xd), np.asarray(wd)
            largest = [max(abs(int(a.max())), abs(int(a.min()))) for a in (xd, wd)]
            if largest[0] * largest[1] * int(np.prod(wd.shape[1:])) >= 2**53:
                raise TypeError(
                    f"conv_nd of integer operands runs in float64 on the GPU, which is exact while no sum can reach 2**53; "
                    f"values up to {largest[0]} and {largest[1]} over {int(np.prod(wd.shape[1:]))} terms may (there is no CPU fallback)"
                )
        grid = tuple(int(g) for g in out_shape)
        out_full = (xd.shape[0], wd.shape[0], *grid)
        self._dtype = dtype
        self._result_dtype = result_dtype
        self._grid = grid
        if xd.size == 0 or wd.size == 0:
            # nothing to gather: every product involves a padding zero
            self._desc = None
            return np.zeros(out_full, dtype=result_dtype) if result_dtype != dtype else _device_zeros(out_full, dtype)

        xb = _device.to_device(xd, dtype)
        wb = _device.to_device(wd, dtype)
        if m > _hip.MG_MAX_ND:
            # more convolved axes than the kernels take: the leading ones are taken apart on the
            # host, tap by tap, into convolutions over the last three (same results, more launches)
            self._desc = "folded"
            ob = _highrank.conv_forward(xb, wb, dtype, tuple(xd.shape), tuple(wd.shape), grid, stride, padding, dilation)
        else:
            self._desc = _hip.shared_desc(_hip.conv_desc, dtype, tuple(xd.shape), tuple(wd.shape), grid, tuple(stride), tuple(padding),
                                          tuple(dilation))
            ob = _device.DeviceBuffer(int(np.prod(out_full)) * dtype.itemsize)
            _hip.check(_hip.lib().mg_conv_fwd(self._desc, xb.ptr, wb.ptr, ob.ptr))
        out, ob = _narrowed(ob, out_full, dtype, result_dtype)
        _device.attach(out, ob)
        return out

    def _complex_forward(self, xd, wd):
        """Complex operands (reference: ``np.tensordot`` multiplies whatever it is given,
        conv.py:96-99; complex arrays reach the operation only under ``no_autodiff``, where the
        reference's own tests take complex-step derivatives through it).  One real convolution
        of twice the channels and filters: with x = a + ib laid out as channels [a, b] and the
        filters as [[p, -q], [q, p]] for w = p + iq, the first F maps of the result are
        a*p - b*q and the last F are a*q + b*p.  Every product stays among parts of its own
        magnitude, which is what a complex step of 1e-20 needs."""
        real = np.float32 if np.result_type(xd.dtype, wd.dtype) == np.complex64 else np.float64
        xd, wd = np.asarray(xd), np.asarray(wd)
        a, b = np.real(xd).astype(real, copy=False), np.imag(xd).astype(real, copy=False)
        p, q = np.real(wd).astype(real, copy=False), np.imag(wd).astype(real, copy=False)
        planes = np.concatenate([a, b], axis=1)
        bank = np.concatenate([np.concatenate([p, -q], axis=1), np.concatenate([q, p], axis=1)], axis=0)
        inner = ConvND()
        both = np.asarray(inner(Tensor(planes, constant=True, copy=False), Tensor(bank, constant=True, copy=False),
                                stride=self.stride, padding=self.padding, dilation=self.dilation))
        filters = wd.shape[0]
        out = np.empty((both.shape[0], filters, *both.shape[2:]), dtype=np.result_type(xd.dtype, wd.dtype))
        out.real = both[:, :filters]
        out.imag = both[:, filters:]
        self._desc = None
        self._dtype = self._result_dtype = out.dtype
        return out

    def backward_var(self, grad, index, **kwargs):
        x, w = (_device.value_of(v) for v in self.variables)
        dtype = self._dtype
        if self._desc is None:
            return np.zeros((x if index == 0 else w).shape, dtype=self._result_dtype) if self._result_dtype != dtype else _device_zeros(
                (x if index == 0 else w).shape, dtype)
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
            out, db = _narrowed(db, x.shape, dtype, self._result_dtype)
        else:  # dw
            xb = _device.to_device(x, dtype)
            if self._desc == "folded":
                db = _highrank.conv_wgrad(gb, xb, *folded)
            else:
                db = _device.DeviceBuffer(w.size * dtype.itemsize)
                _hip.check(lib.mg_conv_wgrad(self._desc, gb.ptr, xb.ptr, db.ptr))
            out, db = _narrowed(db, w.shape, dtype, self._result_dtype)
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
