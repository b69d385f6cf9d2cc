"""``max_pool`` on the MI355X: the MaxPoolND operation with the reference's
signature, argument checks and errors (``mygrad/nnet/layers/pooling.py``),
whose forward pass and gradient routing run as bandwidth-bound kernels in
``libmygrad_hip.so``."""

from math import prod
from numbers import Integral

import numpy as np

from ... import _device, _hip
from ...operation_base import Operation
from ...tensor_base import Tensor

__all__ = ["max_pool", "MaxPoolND"]


class _Stage:
    """One launch's worth of pooling: ``lead`` stacked arrays of shape ``shape`` (one to three
    axes), window ``pool`` placed every ``stride``.  Keeps the argmax bytes of its forward pass
    (windows of up to 256 elements) and, when it is not the first stage, the buffer it read."""

    def __init__(self, lead, shape, pool, stride):
        self.lead = int(lead)
        self.shape = tuple(int(n) for n in shape)
        self.pool = tuple(int(n) for n in pool)
        self.stride = tuple(int(n) for n in stride)
        self.grid = tuple((n - w) // s + 1 for n, w, s in zip(self.shape, self.pool, self.stride))
        self.windows = self.lead * prod(self.grid)
        self.count = self.lead * prod(self.shape)
        self.keeps_argmax = prod(self.pool) <= 256  # what one byte per window can tell apart
        self.argmax = None
        self.source = None  # the device buffer read by the forward pass (stages after the first)

    def desc(self, dtype, dx_dtype=None):
        return _hip.shared_desc(_hip.pool_desc, dtype, self.lead, self.shape, self.pool, self.stride, self.grid, dx_dtype=dx_dtype)

    def forward(self, dtype, xb):
        ob = _device.DeviceBuffer(self.windows * dtype.itemsize)
        if self.keeps_argmax:
            # Each window's argmax (pooling.py:109-111) is found here, while x is being read
            # anyway, and kept on the device as one byte per window: the backward pass then
            # needs grad and these bytes only.
            self.argmax = _device.DeviceBuffer(self.windows)
            _hip.check(_hip.lib().mg_maxpool_fwd_argmax(self.desc(dtype), xb.ptr, ob.ptr, self.argmax.ptr))
        else:
            self.argmax = None
            _hip.check(_hip.lib().mg_maxpool_fwd(self.desc(dtype), xb.ptr, ob.ptr))
        return ob

    def backward(self, x_dtype, g_dtype, gb, dx_dtype, xb, argmax_valid):
        """Routes ``gb`` (values of ``g_dtype``) to a new buffer of ``dx_dtype`` values."""
        db = _device.DeviceBuffer(self.count * dx_dtype.itemsize)
        if self.argmax is not None and argmax_valid:
            _hip.check(_hip.lib().mg_maxpool_bwd_argmax(self.desc(g_dtype, dx_dtype), self.argmax.ptr, gb.ptr, db.ptr))
        else:  # find the maxima again in what the forward pass read
            _hip.check(_hip.lib().mg_maxpool_bwd(self.desc(x_dtype, dx_dtype), xb.ptr, gb.ptr, db.ptr))
        return db


def plan_stages(lead, pooled, pool, stride, most=_hip.MG_MAX_ND):
    """The stages of a pooling over any number of axes, in the order the forward pass runs them:
    the last ``most`` axes first, with everything in front of them counted as leading axes; their
    grid then merges into one axis with a window of one element, and so on until at most ``most``
    axes are left."""
    stages = []
    shape, window, step = [int(n) for n in pooled], [int(n) for n in pool], [int(n) for n in stride]
    while len(shape) > most:
        stage = _Stage(int(lead) * prod(shape[:-most]), shape[-most:], window[-most:], step[-most:])
        stages.append(stage)
        shape = shape[:-most] + [prod(stage.grid)]
        window, step = window[:-most] + [1], step[:-most] + [1]
    stages.append(_Stage(lead, shape, window, step))
    return stages


class MaxPoolND(Operation):
    """Max-pooling over the trailing ``len(pool)`` axes of ``x``.

    ``(N0, ..., C0, ...) -> (N0, ..., G0, ...)`` with window ``(P0, ...)`` placed
    every ``(S0, ...)``; only placements that fit entirely inside the data.

    The kernels pool over one to three axes.  More pooled axes are taken three at a time, from
    the last: the maximum over a window is the maximum, over its leading axes, of the maxima
    over its last three, and the first maximum in row-major order is found the same way (the
    first leading position that holds the maximum, then the first place inside it).  So the
    last three axes are pooled with all others counted as leading axes, the three resulting
    grid axes are merged into one with a window of one element, and the rest is pooled again.
    With two or three stages (four to seven pooled axes) the gradient is routed through all
    records at once, every element adding its windows in the reference's order (bit-exact); with
    more, it takes the stages in reverse, in float64 between them as the reference accumulates it
    (pooling.py:147): the same terms in another order.
    """

    takes_device_arrays = True

    _stages = ()
    _skip = 0  # leading pooled axes with a one-element window, counted as leading axes

    @property
    def _argmax(self):
        """Argmax bytes of the forward pass (of its one stage, for up to three pooled axes)."""
        return self._stages[0].argmax if self._stages else None

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
        if m == 0:
            raise NotImplementedError("max_pool on the GPU needs at least one pooled axis (no CPU fallback)")

        # Leading pooled axes with a window of one element placed at every position pool nothing:
        # they count as un-pooled leading axes.
        skip = 0
        while m - skip > 1 and pool[skip] == 1 and stride[skip] == 1:
            skip += 1
        self._skip = skip
        result_dtype = xd.dtype
        if xd.dtype.kind in "iu":
            # Integers (constants: no gradient is ever asked for) are pooled as float64, which holds
            # every integer below 2**53; a maximum is one of the inputs, so the way back is exact.
            xd = np.asarray(xd)
            if xd.size and max(abs(int(xd.max())), abs(int(xd.min()))) >= 2**53:
                raise TypeError("max_pool of integers runs in float64 on the GPU, which holds integers below 2**53 only "
                                "(there is no CPU fallback)")
            xd = xd.astype(np.float64)
        if xd.dtype not in (np.float32, np.float64, np.float16):
            raise TypeError(
                f"max_pool runs on the GPU in float32 or float64 (float16 values are widened to float32), got {xd.dtype} "
                "(there is no CPU fallback)"
            )
        # float16 is a storage type here: the values are widened to float32 (exactly), the kernels
        # pick the same maxima, and the result is narrowed again (exactly: it consists of inputs)
        if xd.dtype == np.float16:
            xd = xd.astype(np.float32)  # on the device for a value that lives there, else on the host
        grid = tuple(int(g) for g in out_shape)
        self._grid = grid
        self._lead = prod(int(n) for n in lead_shape)
        out_full = (*lead_shape, *grid)
        if self._lead == 0:
            return np.empty(out_full, dtype=result_dtype)

        self._lead *= prod(int(n) for n in pooled[:skip])
        stages = plan_stages(self._lead, pooled[skip:], pool[skip:], stride[skip:])
        self._stages = stages

        buf = _device.to_device(xd)
        for i, stage in enumerate(stages):
            if i:
                stage.source = buf
            buf = stage.forward(xd.dtype, buf)
        if result_dtype != xd.dtype:
            buf = _device.DeviceArray(buf, out_full, xd.dtype).astype(result_dtype).buf
        out = _device.download(buf, out_full, result_dtype)
        _device.attach(out, buf)
        return out

    def backward_var(self, grad, index, **kwargs):
        var = self.variables[index]
        x = _device.value_of(var)
        if self._lead == 0:
            return np.zeros(x.shape, dtype=np.float64)
        held = x  # what the graph holds (and locks)
        half = x.dtype == np.float16
        if half:
            x = x.astype(np.float32)
        if grad.shape != (*x.shape[: x.ndim - len(self.pool)], *self._grid):
            raise ValueError(f"max_pool backward: gradient of shape {grad.shape} for an output of shape "
                             f"{(*x.shape[: x.ndim - len(self.pool)], *self._grid)}")
        # The reference builds dx in float64 whatever x is (pooling.py:147) and the
        # caller rounds it to x.dtype when it becomes var.grad.  The kernel sums in
        # double and rounds once, so it can write x.dtype directly -- except when
        # var already holds a gradient that this one is added to, where the
        # unrounded float64 values are needed for the same result.
        # A float16 x gets the float64 sums, which the caller rounds to float16 in one step.
        dx_dtype = np.dtype(np.float64) if var._grad is not None or half else x.dtype
        wide = np.dtype(np.float64)
        stages = self._stages
        # x is read-only for as long as the graph holds it, so the recorded positions cannot go
        # stale; if it was released and may have been written to, the maxima are found again
        # (for several stages: all of them, from the values x holds now)
        fresh = _device.is_locked(held)
        xb = None
        if not fresh or stages[0].argmax is None:
            xb = _device.to_device(x)
        if not fresh and len(stages) > 1:
            buf = xb
            for i, stage in enumerate(stages):
                if i:
                    stage.source = buf
                buf = stage.forward(x.dtype, buf)
            fresh = True
        gb = _device.to_device(grad, x.dtype)
        g_dtype = x.dtype
        if len(stages) in (2, 3) and fresh and all(stage.argmax is not None for stage in stages):
            # Four to seven pooled axes: the stages' records together name the element a whole window
            # routes to, and one gather adds every element's windows in the row-major order of the
            # whole windows -- np.add.at's order (pooling.py:147-148), bit for bit.  (Stage by stage,
            # as below, the same terms are added in another order.)
            inner = stages[0]
            db = _device.DeviceBuffer(inner.count * dx_dtype.itemsize)
            descs = [stage.desc(x.dtype, dx_dtype) for stage in stages]
            records = [stage.argmax.ptr for stage in stages]
            entry = _hip.lib().mg_maxpool_bwd_argmax_staged if len(stages) == 2 else _hip.lib().mg_maxpool_bwd_argmax_staged3
            _hip.check(entry(*descs, *records, gb.ptr, db.ptr))
            out = _device.download(db, x.shape, dx_dtype)
            _device.attach_transient(out, db)
            return out
        for i in range(len(stages) - 1, -1, -1):
            stage = stages[i]
            last = i == 0
            # between the stages the gradient stays in float64 when the stage can route it from its
            # argmax bytes (the kernels read x and grad in one precision)
            out_dtype = dx_dtype if last else (wide if stages[i - 1].argmax is not None else x.dtype)
            target = out_dtype
            if g_dtype != x.dtype and out_dtype != wide:
                target = wide  # a float64 gradient is routed to float64 and rounded afterwards
            source = xb if last else stage.source
            db = stage.backward(x.dtype, g_dtype, gb, target, source, fresh)
            if target != out_dtype:
                narrow = _device.DeviceBuffer(stage.count * out_dtype.itemsize)
                _hip.check(_hip.lib().mg_cast(_hip.dtype_code(target), _hip.dtype_code(out_dtype), stage.count, db.ptr, narrow.ptr))
                db = narrow
            gb, g_dtype = db, out_dtype
        out = _device.download(gb, x.shape, dx_dtype)
        _device.attach_transient(out, gb)
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
