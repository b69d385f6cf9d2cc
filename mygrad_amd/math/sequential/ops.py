"""``Sum`` over all elements on the MI355X (reference:
``mygrad/math/sequential/ops.py:120-133`` and ``Sequential.__call__``,
``mygrad/operation_base.py:400-470``).

The forward pass is ``np.sum(a)``; the gradient of a full reduction is the incoming
scalar written to every element (``np.full(a.shape, grad, dtype=a.dtype)``).  Reductions
over a subset of the axes are not part of this build and raise."""

import numpy as np

from ... import _device, _hip
from ...operation_base import Operation

__all__ = ["Sum"]


class Sum(Operation):
    def __call__(self, a, axis=None, keepdims=False):
        self.variables = (a,)
        x = a.data
        if axis is not None and not (x.ndim == 0 and axis in ((), (0,))):
            full = tuple(sorted(ax % max(x.ndim, 1) for ax in (axis if hasattr(axis, "__iter__") else (axis,))))
            if full != tuple(range(x.ndim)):
                raise NotImplementedError(
                    f"sum on the GPU reduces over all axes, got axis={axis} for shape {x.shape} (no CPU fallback)"
                )
        if x.dtype not in (np.float32, np.float64):
            raise TypeError(f"sum runs on the GPU in float32 or float64, got {x.dtype} (there is no CPU fallback)")
        self.axis, self.keepdims = None, bool(keepdims)
        out_shape = (1,) * x.ndim if keepdims else ()
        if x.size == 0:
            return np.zeros(out_shape, dtype=x.dtype)
        xb = _device.to_device(x)
        ob = _device.DeviceBuffer(16)
        _hip.check(_hip.lib().mg_sum_all(_hip.dtype_code(x.dtype), x.size, xb.ptr, ob.ptr))
        out = _device.download(ob, out_shape, x.dtype)
        _device.attach(out, ob)
        return out

    def backward_var(self, grad, index, **kwargs):
        (a,) = self.variables
        x = a.data
        grad = np.asarray(grad)
        if grad.size != 1:
            raise NotImplementedError(f"sum backward expects a scalar gradient, got shape {grad.shape}")
        if x.size == 0:
            return np.zeros(x.shape, dtype=x.dtype)
        gb = _device.to_device(np.ascontiguousarray(grad).reshape(()), x.dtype)
        ob = _device.DeviceBuffer(max(x.nbytes, 16))
        _hip.check(_hip.lib().mg_fill_from(_hip.dtype_code(x.dtype), x.size, gb.ptr, ob.ptr))
        out = _device.download(ob, x.shape, x.dtype)
        _device.attach_transient(out, ob)
        return out
