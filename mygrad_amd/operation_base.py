"""The Operation contract the kernels plug into.

Counterpart of the reference's ``mygrad/operation_base.py:54-228``: an
operation implements ``__call__(*tensors, **kw) -> numpy.ndarray`` (binding its
input tensors to ``self.variables``) and ``backward_var(grad, index) ->
numpy.ndarray``; ``backward`` walks the inputs, skips constants, checks and
accumulates each gradient.
"""

from abc import ABC, abstractmethod
from numbers import Real

import numpy as np

from . import _device
from .errors import InvalidBackprop, InvalidGradient, SkipGradient

__all__ = ["Operation"]


class Operation(ABC):
    """Base class of differentiable tensor operations."""

    # conv / pool never return views of their inputs
    can_return_view = False

    variables = ()

    # True for operations whose backward_var takes a gradient that is still on the device (a
    # DeviceArray) as it is; any other operation is handed a host array
    takes_device_arrays = False

    # the list of array locks the graph holds on this operation's behalf (None without the
    # memory guard); Tensor._op sets it, and a tensor whose value is copied to the host while
    # the operation is alive appends the lock on that array
    _guarded = None

    # True for operations whose backward_var hands the incoming gradient to a device kernel
    # for more than one input: backward() then uploads it once for all of them
    gradient_on_device = False

    @abstractmethod
    def __call__(self, *input_vars, **kwargs):
        """Forward pass; must bind the tuple of input tensors to ``self.variables``
        and return the result as a NumPy array."""
        raise NotImplementedError()

    @abstractmethod
    def backward_var(self, grad, index, **kwargs):
        """Gradient of the terminal scalar with respect to ``self.variables[index]``
        given ``grad``, its gradient with respect to this operation's output."""
        raise NotImplementedError()

    def backward(self, grad, **kwargs):
        """Back-propagate ``grad`` to every non-constant input
        (reference: operation_base.py:162-228)."""
        if self.gradient_on_device and sum(not var.constant for var in self.variables) > 1:
            _device.hold_gradient(grad)
        for index, var in enumerate(self.variables):
            if var.constant:
                continue

            if not var._ops:
                raise InvalidBackprop(
                    f"Part of the computational graph containing this tensor, {var}, was 'cleared' prior "
                    "to backprop.\nIt is recommended that you clear all computational graphs and restart "
                    "your computation."
                )

            try:
                backed = self.backward_var(grad, index, **kwargs)
            except SkipGradient:
                continue

            if isinstance(backed, _device.DeviceArray):
                if backed.shape == var.shape:
                    self._accumulate_on_device(var, backed, grad)
                    continue
                backed = backed.host()  # a gradient that still has to be summed to var's shape
            if not isinstance(backed, (np.ndarray, np.number, Real)):
                raise InvalidGradient(
                    f"An invalid gradient-value was passed to:\n\t`{type(self).__name__}.backward_var("
                    f"<gradient>, index={index})`\nGradients are expected to be real-valued scalars or "
                    f"numpy arrays, got a gradient of type: {type(backed)}"
                )
            backed = np.asarray(backed)
            if backed.shape != var.shape:
                backed = _sum_to_shape(backed, var.shape)
            assert backed.shape == var.shape, (backed.shape, var.shape)

            if var._grad is None:
                if backed.base is not None and not _is_foreign_buffer(backed) or backed is grad:
                    # a view of something else (or the incoming gradient itself):
                    # the stored gradient must be safe to update in place later
                    mirror = _device.lookup(backed)
                    backed = np.copy(backed)
                    if mirror is not None:
                        _device.attach_transient(backed, mirror)
                if backed.dtype != var.dtype:
                    backed = backed.astype(var.dtype, copy=False)
                var._grad = backed
            else:
                if isinstance(var._grad, _device.DeviceArray):
                    var._grad = var._grad.host()
                _device.evict(var._grad)  # the host copy is about to change
                var._grad += backed

    @staticmethod
    def _accumulate_on_device(var, backed, grad):
        """The same bookkeeping for a gradient that is on the device (and has var's shape):
        copied if it shares its buffer with something else, cast to var's dtype, stored; or
        added into the gradient var already holds (reference: operation_base.py:216-228)."""
        if var._grad is None:
            if backed.base is not None or backed is grad:
                backed = backed.copy()
            if backed.dtype != var.dtype:
                if var.dtype in (np.float32, np.float64, np.float16):
                    backed = backed.astype(var.dtype)
                else:
                    backed = backed.host().astype(var.dtype)
            var._grad = backed
            return
        held = var._grad
        if isinstance(held, _device.DeviceArray) and held._host is None and held.base is None and held.dtype in (np.float32, np.float64, np.float16):
            held.add_into(backed)
            return
        if isinstance(held, _device.DeviceArray):
            held = var._grad = held.host()
        _device.evict(held)  # the host copy is about to change
        held += backed.host()


def _is_foreign_buffer(arr):
    """True for an array that is the direct, whole view of a non-ndarray buffer
    (pinned host memory): it owns its memory as far as NumPy semantics go."""
    return not isinstance(arr.base, np.ndarray) and arr.flags["C_CONTIGUOUS"]


def _sum_to_shape(grad, shape):
    """Sum a broadcast gradient back to ``shape`` (reference:
    mygrad/_utils/__init__.py:131-168)."""
    if grad.ndim < len(shape):
        raise ValueError(f"The dimensionality of the gradient cannot be less than that of its tensor: {grad.shape}, {shape}")
    extra = grad.ndim - len(shape)
    if extra:
        grad = grad.sum(axis=tuple(range(extra)))
    keep = tuple(n for n, i in enumerate(shape) if i == 1 and grad.shape[n] != 1)
    if keep:
        grad = grad.sum(axis=keep, keepdims=True)
    return grad
