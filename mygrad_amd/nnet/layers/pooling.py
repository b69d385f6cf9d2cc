"""``max_pool`` on the MI355X: the MaxPoolND operation with the reference's
signature, argument checks and errors (``mygrad/nnet/layers/pooling.py``),
whose forward pass and gradient routing run as bandwidth-bound kernels in
``libmygrad_hip.so``."""

from numbers import Integral

import numpy as np

from ... import _device, _hip
from ...operation_base import Operation
from ...tensor_base import Tensor

__all__ = ["max_pool", "MaxPoolND"]


class MaxPoolND(Operation):
    """Max-pooling over the trailing ``len(pool)`` axes of ``x``.

    ``(N0, ..., C0, ...) -> (N0, ..., G0, ...)`` with window ``(P0, ...)`` placed
    every ``(S0, ...)``; only placements that fit entirely inside the data.
    """

    takes_device_arrays = True

    _argmax = None  # device buffer, one byte per window, written by the forward pass
    _skip = 0  # leading pooled axes with a one-element window, counted as leading axes

    def __call__(self, x, pool, stride):
        self.variables = (x,)
        xd = _device.value_of(x)

        assert isinstance(pool, (tuple, list, np.ndarray)) and all(
            i >= 0 and isinstance(i, Integral) for i in pool
        )
        pool = np.asarray(pool, dtype=int)
        assert all(i > 0 for i in pool)
        assert xd.ndim >= len(
            pool
        ), "The number of pooled dimensions cannot exceed the dimensionality of the data."
        stride = (
            np.array([stride] * len(pool)) if isinstance(stride, Integral) else np.asarray(stride, dtype=int)
        )
        assert len(stride) == len(pool) and all(s >= 1 and isinstance(s, Integral) for s in stride)

        self.pool, self.stride = pool, stride
        m = len(pool)
        lead_shape = xd.shape[: xd.ndim - m]
        pooled = np.array(xd.shape[xd.ndim - m :])

        out_shape = (pooled - pool) / stride + 1
        if not all(i.is_integer() and i > 0 for i in out_shape):
            raise ValueError(
                "Stride and kernel dimensions are incompatible: \n"
                f"Input dimensions: {tuple(pooled)}\n"
                f"Stride dimensions: {tuple(stride)}\n"
                f"Pooling dimensions: {tuple(pool)}\n"
            )

        # Leading pooled axes with a window of one element placed at every position pool nothing:
        # they count as un-pooled leading axes.  What is left must fit the kernels' three axes.
        skip = 0
        while m - skip > _hip.MG_MAX_ND and pool[skip] == 1 and stride[skip] == 1:
            skip += 1
        if not 1 <= m - skip <= _hip.MG_MAX_ND:
            raise NotImplementedError(
                f"max_pool on the GPU handles 1 to {_hip.MG_MAX_ND} pooled axes (leading axes with a window of one "
                f"element aside), got pool={tuple(pool)} stride={tuple(stride)} (no CPU fallback)"
            )
        self._skip = skip
        if xd.dtype not in (np.float32, np.float64):
            raise TypeError(
                f"max_pool runs on the GPU in float32 or float64, got {xd.dtype} (there is no CPU fallback)"
            )
        grid = tuple(int(g) for g in out_shape)
        self._grid = grid
        self._lead = int(np.prod(lead_shape, dtype=np.int64))
        out_full = (*lead_shape, *grid)
        if self._lead == 0:
            return np.empty(out_full, dtype=xd.dtype)

        self._lead *= int(np.prod(pooled[:skip], dtype=np.int64))
        desc = _hip.pool_desc(xd.dtype, self._lead, pooled[skip:], pool[skip:], stride[skip:], grid[skip:])
        xb = _device.to_device(xd)
        windows = int(np.prod(out_full))
        ob = _device.DeviceBuffer(windows * xd.dtype.itemsize)
        if int(np.prod(pool)) <= 256:
            # Each window's argmax (pooling.py:109-111) is found here, while x is being read
            # anyway, and kept on the device as one byte per window: the backward pass then
            # needs grad and these bytes only.  x is read-only for as long as the graph holds
            # it, so the positions cannot go stale; backward_var checks that this still holds.
            self._argmax = _device.DeviceBuffer(windows)
            _hip.check(_hip.lib().mg_maxpool_fwd_argmax(desc, xb.ptr, ob.ptr, self._argmax.ptr))
        else:
            _hip.check(_hip.lib().mg_maxpool_fwd(desc, xb.ptr, ob.ptr))
        out = _device.download(ob, out_full, xd.dtype)
        _device.attach(out, ob)
        return out

    def backward_var(self, grad, index, **kwargs):
        var = self.variables[index]
        x = _device.value_of(var)
        if self._lead == 0:
            return np.zeros(x.shape, dtype=np.float64)
        if grad.shape != (*x.shape[: x.ndim - len(self.pool)], *self._grid):
            raise ValueError(f"max_pool backward: gradient of shape {grad.shape} for an output of shape "
                             f"{(*x.shape[: x.ndim - len(self.pool)], *self._grid)}")
        m = len(self.pool)
        # The reference builds dx in float64 whatever x is (pooling.py:147) and the
        # caller rounds it to x.dtype when it becomes var.grad.  The kernel sums in
        # double and rounds once, so it can write x.dtype directly -- except when
        # var already holds a gradient that this one is added to, where the
        # unrounded float64 values are needed for the same result.
        dx_dtype = np.dtype(np.float64) if var._grad is not None else x.dtype
        k = self._skip
        desc = _hip.pool_desc(x.dtype, self._lead, x.shape[x.ndim - m + k :], self.pool[k:], self.stride[k:], self._grid[k:],
                              dx_dtype=dx_dtype)
        gb = _device.to_device(grad, x.dtype)
        db = _device.DeviceBuffer(x.size * dx_dtype.itemsize)
        if self._argmax is not None and _device.is_locked(x):
            _hip.check(_hip.lib().mg_maxpool_bwd_argmax(desc, self._argmax.ptr, gb.ptr, db.ptr))
        else:  # x may have been written to since the forward pass: find the maxima again
            xb = _device.to_device(x)
            _hip.check(_hip.lib().mg_maxpool_bwd(desc, xb.ptr, gb.ptr, db.ptr))
        out = _device.download(db, x.shape, dx_dtype)
        _device.attach_transient(out, db)
        return out


def max_pool(x, pool, stride, *, constant=None):
    """Perform max-pooling over the last N dimensions of a data batch.

    The data has N trailing axes to be pooled over, ``(C0, ...)``, optionally
    preceded by un-pooled axes ``(N0, ...)``.  The window ``(P0, ...)`` is placed
    with strides ``(S0, ...)``; the pooled axes come out with shape ``(G0, ...)``.

    Parameters
    ----------
    x : ArrayLike, shape=([...], C0, ...)
        The data batch; pooled along its trailing axes.
    pool : Tuple[int, ...], (P0, ...)
        Extent of the pooling window; its length is the number of pooled axes.
    stride : Union[int, Tuple[int, ...]], (S0, ...)
        Spacing of the window placements; one value is used for all pooled axes.
    constant : Optional[bool]
        If True, the resulting Tensor is a constant.

    Returns
    -------
    Tensor, shape=([...], G0, ...)

    Raises
    ------
    ValueError
        ``(C - P) / S + 1`` is not a positive integer along some pooled axis.
    AssertionError
        ``pool`` / ``stride`` has the wrong type, length or a non-positive value.

    Notes
    -----
    Where several elements of a window share the maximum, the gradient goes to
    the first of them in row-major order.

    Examples
    --------
    >>> from mygrad_amd import Tensor
    >>> from mygrad_amd.nnet import max_pool
    >>> x = Tensor([[0., 10., 8.], [2., 7., 3.], [5., 7., 20.]])
    >>> out = max_pool(x, pool=(2, 2), stride=1)
    >>> out.backward()
    >>> x.grad
    array([[0., 2., 0.],
           [0., 1., 0.],
           [0., 0., 1.]])
    """
    return Tensor._op(MaxPoolND, x, op_args=(pool, stride), constant=constant)
