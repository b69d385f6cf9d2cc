"""``relu`` on the MI355X (reference: ``mygrad/nnet/activations/relu.py``).

``f(x) = x * (x > 0)`` computed, like the reference, as a multiplication by a 0/1 mask:
negative inputs give ``-0.0`` and NaN stays NaN.  The mask the reference keeps in
``self.back`` is kept here as well, on the device, as one bit per element: the backward
kernel reads the gradient and the bits, not ``x``."""

import numpy as np

from ... import _device, _hip
from ...operation_base import Operation
from ...tensor_base import Tensor

__all__ = ["relu", "ReLu"]


class ReLu(Operation):
    takes_device_arrays = True

    def __call__(self, a):
        self.variables = (a,)
        x = _device.value_of(a)
        if x.dtype not in (np.float32, np.float64):
            raise TypeError(f"relu runs on the GPU in float32 or float64, got {x.dtype} (there is no CPU fallback)")
        if x.size == 0:
            return np.empty(x.shape, dtype=x.dtype)
        xb = _device.to_device(x)
        ob = _device.DeviceBuffer(max(x.nbytes, 16))
        self._mask = _device.DeviceBuffer(max((x.size + 7) // 8, 16))  # the reference's self.back, packed
        _hip.check(_hip.lib().mg_relu_fwd_mask(_hip.dtype_code(x.dtype), x.size, xb.ptr, ob.ptr, self._mask.ptr))
        out = _device.download(ob, x.shape, x.dtype)
        _device.attach(out, ob)
        return out

    def backward_var(self, grad, index, **kwargs):
        x = _device.value_of(self.variables[index])
        if x.size == 0:
            return np.empty(x.shape, dtype=x.dtype)
        if grad.shape != x.shape:
            raise NotImplementedError(f"relu backward for gradient of shape {grad.shape} (no CPU fallback)")
        gb = _device.to_device(grad, x.dtype)
        ob = _device.DeviceBuffer(max(x.nbytes, 16))
        _hip.check(_hip.lib().mg_relu_bwd_mask(_hip.dtype_code(x.dtype), x.size, self._mask.ptr, gb.ptr, ob.ptr))
        out = _device.download(ob, x.shape, x.dtype)
        _device.attach_transient(out, ob)
        return out


def relu(x, *, constant=None):
    """Applies the rectified linear unit activation function::

        f(x) = {x, x > 0
                0, x <= 0 }

    Parameters
    ----------
    x : ArrayLike
        relu is applied element-wise on ``x``.
    constant : Optional[bool]
        If True, the returned tensor is a constant.

    Returns
    -------
    Tensor

    Examples
    --------
    >>> import mygrad_amd as mg
    >>> from mygrad_amd.nnet import relu
    >>> x = mg.Tensor([-5., -2.5, 0., 2.5, 5.])
    >>> relu(x)
    Tensor([-0. , -0. ,  0. ,  2.5,  5. ])
    >>> relu(x).backward()
    >>> x.grad
    array([0., 0., 0., 1., 1.])
    """
    return Tensor._op(ReLu, x, constant=constant)
