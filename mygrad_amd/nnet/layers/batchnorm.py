"""``batchnorm`` on the MI355X: the BatchNorm operation with the reference's signature
and attributes (``mygrad/nnet/layers/batchnorm.py``), whose statistics, normalisation and
gradients run as bandwidth-bound kernels in ``libmygrad_hip.so``.

The reference keeps the normalised batch in ``self.x_norm`` for the backward pass; here it
is recomputed on the device from ``x``, ``mean`` and ``var`` (one subtraction and one
division per element), which saves holding a second copy of the batch."""

from typing import Optional

import numpy as np

from ... import _device, _hip
from ...operation_base import Operation
from ...tensor_base import Tensor

__all__ = ["batchnorm", "BatchNorm"]


class BatchNorm(Operation):
    """Per-channel normalisation with optional scale and shift.  Calling the instance binds
    the channel statistics it computed as ``self.mean`` and ``self.var`` (each ``(C,)``)."""

    takes_device_arrays = True

    def __call__(self, x, gamma, beta, *, eps):
        """``x:(N, C, ...)``; ``gamma`` / ``beta``: ``(C,)`` tensors, or empty ones for "no
        scale" / "no shift" (how the wrapper passes ``None``); returns the normalised array."""
        self.variables = tuple(i for i in (x, gamma, beta))

        if gamma.size == 0:
            gamma = None
        if beta.size == 0:
            beta = None

        self.gamma = gamma
        self.beta = beta
        self.eps = float(eps)

        xd = _device.value_of(x)
        if xd.ndim < 2:
            raise ValueError(f"batchnorm normalises every axis but axis 1: `x` must have at least 2 axes, got shape {xd.shape}")
        if xd.dtype not in (np.float32, np.float64):
            raise TypeError(f"batchnorm runs on the GPU in float32 or float64, got {xd.dtype} (there is no CPU fallback)")
        channels = xd.shape[1]
        for name, t in (("gamma", gamma), ("beta", beta)):
            if t is None:
                continue
            if _device.value_of(t).shape != (channels,):
                raise ValueError(f"`{name}` must have shape ({channels},), got {_device.value_of(t).shape}")
            if _device.value_of(t).dtype != xd.dtype:
                raise TypeError(
                    f"batchnorm on the GPU takes `{name}` in the dtype of `x` ({xd.dtype}), got {_device.value_of(t).dtype}"
                )
        if not self.eps >= 0:
            raise ValueError(f"`eps` must be a non-negative number, got {eps}")

        self._bwd = None
        if xd.size == 0:
            self._mean = np.full((channels,), np.nan, dtype=xd.dtype)
            self._var = np.full((channels,), np.nan, dtype=xd.dtype)
            return np.empty(xd.shape, dtype=xd.dtype)

        desc = self._desc = _hip.bn_desc(xd.shape, xd.dtype, gamma is not None, beta is not None, self.eps)
        xb = _device.to_device(xd)
        gb = _device.to_device(_device.value_of(gamma)) if gamma is not None else None
        bb = _device.to_device(_device.value_of(beta)) if beta is not None else None
        yb = _device.DeviceBuffer(max(xd.nbytes, 16))
        self._mean_dev = _device.DeviceBuffer(max(channels * xd.itemsize, 16))
        self._var_dev = _device.DeviceBuffer(max(channels * xd.itemsize, 16))
        _hip.check(
            _hip.lib().mg_batchnorm_fwd(
                desc,
                xb.ptr,
                gb.ptr if gb is not None else None,
                bb.ptr if bb is not None else None,
                yb.ptr,
                self._mean_dev.ptr,
                self._var_dev.ptr,
            )
        )
        # copied to the host when somebody asks for them (the backward pass reads the device copies)
        self._mean = _device.DeviceArray(self._mean_dev, (channels,), xd.dtype)
        self._var = _device.DeviceArray(self._var_dev, (channels,), xd.dtype)
        y = _device.download(yb, xd.shape, xd.dtype)
        _device.attach(y, yb)
        return y

    @property
    def mean(self):
        """Per-channel mean of the batch (the reference's ``self.mean``, batchnorm.py:57)."""
        if isinstance(self._mean, _device.DeviceArray):
            self._mean = self._mean.host()
        return self._mean

    @property
    def var(self):
        """Per-channel (biased) variance of the batch (the reference's ``self.var``, batchnorm.py:58)."""
        if isinstance(self._var, _device.DeviceArray):
            self._var = self._var.host()
        return self._var

    def _run_backward(self, grad, want):
        """One pass over (x, grad) for every gradient in ``want`` (a set of "x", "gamma",
        "beta"); returns them as a dict of arrays."""
        x = _device.value_of(self.variables[0])
        channels = x.shape[1]
        if grad.shape != x.shape:
            raise NotImplementedError(f"batchnorm backward for gradient of shape {grad.shape} (no CPU fallback)")
        xb = _device.to_device(x)
        gradb = _device.to_device(grad, x.dtype)
        gb = _device.to_device(_device.value_of(self.gamma)) if self.gamma is not None else None
        small = max(channels * x.itemsize, 16)
        dxb = _device.DeviceBuffer(max(x.nbytes, 16)) if "x" in want else None
        dgb = _device.DeviceBuffer(small) if "gamma" in want else None
        dbb = _device.DeviceBuffer(small) if "beta" in want else None
        _hip.check(
            _hip.lib().mg_batchnorm_bwd(
                self._desc,
                xb.ptr,
                gradb.ptr,
                gb.ptr if gb is not None else None,
                self._mean_dev.ptr,
                self._var_dev.ptr,
                dxb.ptr if dxb is not None else None,
                dgb.ptr if dgb is not None else None,
                dbb.ptr if dbb is not None else None,
            )
        )
        out = {}
        if dxb is not None:
            out["x"] = _device.download(dxb, x.shape, x.dtype)
            _device.attach_transient(out["x"], dxb)
        if dgb is not None:
            out["gamma"] = _device.download(dgb, (channels,), x.dtype)
        if dbb is not None:
            out["beta"] = _device.download(dbb, (channels,), x.dtype)
        return out

    def _which(self, index):
        if index == 0:
            return "x"
        if index == 1 and self.gamma is not None:
            return "gamma"
        if (index == 1 and self.gamma is None) or index == 2:
            return "beta"
        raise IndexError

    def backward_var(self, grad, index, **kwargs):
        which = self._which(index)
        x = _device.value_of(self.variables[0])
        if x.size == 0:
            return np.zeros(x.shape if which == "x" else (x.shape[1],), dtype=x.dtype)
        # backward() asks for each variable in turn with the same `grad`: the first request
        # computes everything the graph needs in one pass over the batch
        if self._bwd is None or self._bwd[0] is not grad or which not in self._bwd[1]:
            want = {which}
            for i, var in enumerate(self.variables):
                if var.size and not var.constant:
                    want.add(self._which(i))
            self._bwd = (grad, self._run_backward(grad, want))
        out = self._bwd[1].pop(which)
        if not self._bwd[1]:
            self._bwd = None
        return out


def batchnorm(
    x,
    *,
    gamma=None,
    beta=None,
    eps: float,
    constant: Optional[bool] = None,
) -> Tensor:
    """Normalise ``x:(N, C, ...)`` per channel (axis 1) over all other axes, on the GPU::

        batchnorm(x) = gamma * (x - mean_c) / sqrt(var_c + eps) + beta

    ``gamma`` and ``beta`` are optional ``(C,)`` tensors in the dtype of ``x`` (float32 or
    float64); ``eps`` is a non-negative number and has no default; ``constant=True`` makes
    the result a constant.  The operation keeps the channel statistics as ``.mean`` and
    ``.var`` (``y.creator.mean``) like the reference.

    >>> import mygrad_amd as mg
    >>> from mygrad_amd.nnet import batchnorm
    >>> batchnorm(mg.Tensor([[1.], [4.], [1.]]), eps=0).data.ravel()
    array([-0.70710678,  1.41421356, -0.70710678])
    """
    # gamma and beta travel as empty arrays when they are not supplied
    if gamma is None:
        gamma = np.array([])
    if beta is None:
        beta = np.array([])
    return Tensor._op(BatchNorm, x, gamma, beta, op_kwargs=dict(eps=eps), constant=constant)
