"""``Multiply`` on the MI355X (reference: ``mygrad/math/arithmetic/ops.py:45-53``).

The reference's ``Multiply`` is ``np.multiply`` with broadcasting and gradients
``grad * other``.  This build runs the case that occurs between the convolution /
pooling kernels -- two operands of the same shape and floating-point dtype -- as one
bandwidth-bound kernel; other argument patterns raise (there is no CPU fallback)."""

import numpy as np

from ... import _device, _hip
from ...operation_base import Operation

__all__ = ["Multiply"]


def _same_shape_floats(op, a, b):
    if a.shape != b.shape:
        raise NotImplementedError(
            f"{op} on the GPU takes operands of one shape, got {a.shape} and {b.shape} "
            "(broadcasting is not part of this build; there is no CPU fallback)"
        )
    dtype = np.result_type(a, b)
    if dtype not in (np.float32, np.float64):
        raise TypeError(f"{op} runs on the GPU in float32 or float64, got {a.dtype} and {b.dtype} (there is no CPU fallback)")
    return np.dtype(dtype)


def device_multiply(a, b, dtype):
    """``a * b`` for two same-shape host arrays -> (host result, its device buffer)."""
    ab, bb = _device.to_device(a, dtype), _device.to_device(b, dtype)
    ob = _device.DeviceBuffer(max(a.size * dtype.itemsize, 16))
    _hip.check(_hip.lib().mg_multiply(_hip.dtype_code(dtype), a.size, ab.ptr, bb.ptr, ob.ptr))
    return _device.download(ob, a.shape, dtype), ob


class Multiply(Operation):
    """``f(a, b) -> a * b`` element-wise."""

    gradient_on_device = True

    def __call__(self, a, b):
        self.variables = (a, b)
        dtype = _same_shape_floats("multiply", a.data, b.data)
        self._dtype = dtype
        out, ob = device_multiply(a.data, b.data, dtype)
        _device.attach(out, ob)
        return out

    def backward_var(self, grad, index, **kwargs):
        a, b = self.variables
        other = b.data if index == 0 else a.data
        dtype = np.dtype(np.result_type(grad, other))
        if grad.shape != other.shape or dtype not in (np.float32, np.float64):
            raise NotImplementedError(f"multiply backward for gradient {grad.shape} {grad.dtype} (no CPU fallback)")
        out, ob = device_multiply(grad, other, dtype)
        _device.attach_transient(out, ob)
        return out
