"""``Multiply`` on the MI355X (reference: ``mygrad/math/arithmetic/ops.py:45-53``).

The reference's ``Multiply`` is ``np.multiply`` with broadcasting and gradients
``grad * other``, summed back to the operand's shape over the axes it was broadcast along
(``mygrad/_utils/__init__.py:131-168``).  Operands of one shape -- the case between the
convolution / pooling kernels -- take one bandwidth-bound kernel; so do operands that are
broadcast (``mg_multiply_broadcast`` reads each where it lies; only a pattern with more than
six groups of axes is first spread to the common shape on the device), and the gradient of a
broadcast operand is summed back on the device (carried in double, rounded once: equal to
NumPy's pairwise sum to rounding).
Floating-point operands only; other argument patterns raise (there is no CPU fallback)."""

import numpy as np

from ... import _device, _hip, _reduce
from ...operation_base import Operation

__all__ = ["Multiply"]


def _float_dtype(op, a, b):
    dtype = np.result_type(a.dtype, b.dtype)
    if dtype not in (np.float32, np.float64):
        raise TypeError(f"{op} runs on the GPU in float32 or float64, got {a.dtype} and {b.dtype} (there is no CPU fallback)")
    return np.dtype(dtype)


def _spread(arr, shape, dtype):
    """Device buffer with ``arr`` cast to ``dtype`` and broadcast to ``shape``."""
    buf = _device.to_device(arr, dtype)
    return buf if arr.shape == tuple(shape) else _reduce.broadcast(buf, arr.shape, shape, dtype)


def device_multiply(a, b, dtype, shape=None):
    """``a * b`` for two host arrays that broadcast to ``shape`` -> (host result, its device buffer)."""
    shape = a.shape if shape is None else tuple(shape)
    size = int(np.prod(shape, dtype=np.int64))
    if size == 0:
        return np.empty(shape, dtype=dtype), None
    ob = None
    if a.shape != shape or b.shape != shape:
        # one pass that reads each operand where it lies
        ob = _reduce.multiply_broadcast(_device.to_device(a, dtype), a.shape, _device.to_device(b, dtype), b.shape, shape, dtype)
    if ob is None:
        ab, bb = _spread(a, shape, dtype), _spread(b, shape, dtype)
        ob = _device.DeviceBuffer(max(size * dtype.itemsize, 16))
        _hip.check(_hip.lib().mg_multiply(_hip.dtype_code(dtype), size, ab.ptr, bb.ptr, ob.ptr))
    return _device.download(ob, shape, dtype), ob


class Multiply(Operation):
    """``f(a, b) -> a * b`` element-wise, with NumPy's broadcasting."""

    takes_device_arrays = True

    gradient_on_device = True

    def __call__(self, a, b):
        self.variables = (a, b)
        dtype = _float_dtype("multiply", _device.value_of(a), _device.value_of(b))
        self._dtype = dtype
        self._shape = np.broadcast_shapes(a.shape, b.shape)  # ValueError for shapes that do not go together
        out, ob = device_multiply(_device.value_of(a), _device.value_of(b), dtype, self._shape)
        if ob is not None:
            _device.attach(out, ob)
        return out

    def backward_var(self, grad, index, **kwargs):
        a, b = self.variables
        var, other = (a, b) if index == 0 else (b, a)
        dtype = np.dtype(np.result_type(grad.dtype, other.dtype))
        if grad.shape != self._shape or dtype not in (np.float32, np.float64):
            raise NotImplementedError(f"multiply backward for gradient {grad.shape} {grad.dtype} (no CPU fallback)")
        if var.size == int(np.prod(self._shape, dtype=np.int64)):  # nothing to add up (axes of length one at most)
            out, ob = device_multiply(grad, _device.value_of(other), dtype, self._shape)
            if ob is None:
                return np.zeros(var.shape, dtype=dtype)
            if out.shape != var.shape:
                out = out.reshape(var.shape)  # shares its buffer: the caller copies it before keeping it
            _device.attach_transient(out, ob)
            return out
        if 0 in self._shape:
            return np.zeros(var.shape, dtype=dtype)
        # the operand was broadcast: add its gradient up over the axes it was spread along
        # (reduce_broadcast: the leading axes it lacks and those where it has length one)
        lead = len(self._shape) - var.ndim
        axes = tuple(range(lead)) + tuple(lead + i for i, n in enumerate(var.shape) if n == 1 and self._shape[lead + i] != 1)
        if other.shape == self._shape:
            # product and sums in one pass over the gradient and the other operand
            rb = _reduce.sum_axes(_device.to_device(grad, dtype), self._shape, axes, dtype, times=_device.to_device(_device.value_of(other), dtype))
        else:
            _, ob = device_multiply(grad, _device.value_of(other), dtype, self._shape)
            rb = _reduce.sum_axes(ob, self._shape, axes, dtype)
        back = _device.download(rb, var.shape, dtype)
        _device.attach_transient(back, rb)
        return back
