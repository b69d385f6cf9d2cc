"""``Sum`` on the MI355X (reference: ``mygrad/math/sequential/ops.py:120-133`` and
``Sequential.__call__``, ``mygrad/operation_base.py:400-452``).

The forward pass is ``np.sum(a, axis=axis, keepdims=keepdims)``; the gradient is the
incoming gradient spread back over the summed axes (``np.full`` for a sum over
everything, else ``np.broadcast_to`` after the summed axes have been put back as axes of
length one).  Sums are carried in double on the device and rounded once, where NumPy adds
pairwise in the array's own precision: the results agree to rounding, not bit for bit."""

import numpy as np
from numpy.lib.array_utils import normalize_axis_tuple

from ... import _device, _hip, _reduce
from ...operation_base import Operation

__all__ = ["Sum"]


class Sum(Operation):
    takes_device_arrays = True

    def __call__(self, a, axis=None, keepdims=False):
        self.variables = (a,)
        x = _device.value_of(a)
        # the reference keeps a single axis as a one-tuple (operation_base.py:424-431)
        self.axis = axis if axis is None or hasattr(axis, "__iter__") else (axis,)
        self.keepdims = bool(keepdims)
        if axis is None or x.ndim == 0:
            if x.ndim == 0 and axis is not None:
                normalize_axis_tuple(axis, 1)  # NumPy lets a scalar be summed over axis 0 / -1 / ()
            axes = tuple(range(x.ndim))
        else:
            axes = normalize_axis_tuple(axis, x.ndim)  # the errors np.sum raises for a bad axis
        if x.dtype not in (np.float32, np.float64):
            raise TypeError(f"sum runs on the GPU in float32 or float64, got {x.dtype} (there is no CPU fallback)")
        self._axes = axes
        kept_shape = tuple(1 if i in axes else n for i, n in enumerate(x.shape))
        self._kept_shape = kept_shape
        out_shape = kept_shape if keepdims else tuple(n for i, n in enumerate(x.shape) if i not in axes)
        if int(np.prod(out_shape, dtype=np.int64)) == 0:
            return np.zeros(out_shape, dtype=x.dtype)
        if x.size == 0:  # something is left, nothing to add to it
            return np.zeros(out_shape, dtype=x.dtype)
        xb = _device.to_device(x)
        if len(axes) == x.ndim:
            ob = _device.DeviceBuffer(16)
            _hip.check(_hip.lib().mg_sum_all(_hip.dtype_code(x.dtype), x.size, xb.ptr, ob.ptr))
        else:
            ob = _reduce.sum_axes(xb, x.shape, axes, x.dtype)
            if ob is xb:  # only axes of length one were named: the values are x's own
                ob = _device.DeviceBuffer(max(x.nbytes, 16))
                _hip.check(_hip.lib().mg_memcpy_d2d(ob.ptr, xb.ptr, x.nbytes))
        out = _device.download(ob, out_shape, x.dtype)
        _device.attach(out, ob)
        return out

    def backward_var(self, grad, index, **kwargs):
        (a,) = self.variables
        x = _device.value_of(a)
        if not isinstance(grad, _device.DeviceArray):
            grad = np.ascontiguousarray(grad)
        if x.size == 0:
            return np.zeros(x.shape, dtype=x.dtype)
        lib, code = _hip.lib(), _hip.dtype_code(x.dtype)
        if len(self._axes) == x.ndim:
            if grad.size != 1:
                raise ValueError(f"the gradient of a sum over every axis holds one value, got shape {grad.shape}")
            gb = _device.to_device(grad.reshape(()), x.dtype)
            ob = _device.DeviceBuffer(max(x.nbytes, 16))
            _hip.check(lib.mg_fill_from(code, x.size, gb.ptr, ob.ptr))
        else:
            if grad.size * int(np.prod([x.shape[i] for i in self._axes], dtype=np.int64)) != x.size:
                raise ValueError(f"gradient of shape {grad.shape} does not fit a sum of {x.shape} over axes {self._axes}")
            gb = _device.to_device(grad, x.dtype)
            ob = _reduce.broadcast(gb, self._kept_shape, x.shape, x.dtype)
            if ob is gb:  # nothing to spread: a copy the caller may keep
                ob = _device.DeviceBuffer(max(x.nbytes, 16))
                _hip.check(lib.mg_memcpy_d2d(ob.ptr, gb.ptr, x.nbytes))
        out = _device.download(ob, x.shape, x.dtype)
        _device.attach_transient(out, ob)
        return out
