"""A minimal ``Tensor`` that records the graph of operations and drives
back-propagation through them.

This is the caller side of the Operation contract, restated from the
reference's ``mygrad/tensor_base.py`` (``Tensor._op`` :1022-1212, ``backward``
:1232-1340, ``_backward`` :1342-1378, ``clear_graph`` :1461-1498) and
``mygrad/_utils/__init__.py:36-73`` (topological sort): what `_op` wraps and
locks, how `constant` propagates, how gradients are seeded, accumulated and
cleared.  Views, in-place operations and the NumPy-function overrides of the
reference are outside this path and are not provided.
"""

from collections import deque
from numbers import Integral
from weakref import ReferenceType, finalize

import numpy as np

from . import _device, _graph

__all__ = ["Tensor", "tensor", "asarray", "device_tensor"]

_CONSTANT_ONLY = (np.integer, np.bool_)


def asarray(a, dtype=None):
    """``numpy.asarray`` that unwraps tensors."""
    if isinstance(a, Tensor):
        a = a.data
    return np.asarray(a, dtype=dtype)


def tensor(x, *, dtype=None, constant=None, copy=True, ndmin=0):
    """Create a tensor (counterpart of ``mygrad.tensor``)."""
    return Tensor(x, dtype=dtype, constant=constant, copy=copy, ndmin=ndmin)


def device_tensor(x, *, dtype=None, constant=None):
    """A tensor whose values are uploaded once, now, and live on the device from then on (not a
    function of the reference, whose arrays are all host arrays).

    A tensor made from a host array is uploaded by the first operation that reads it and the
    copy is kept only while a graph holds the array read-only, so a training loop that feeds the
    same host array to a new graph every step uploads it every step.  A device tensor has no host
    array that could change behind the copy: it is never uploaded again, an operation reads it in
    place, and ``.data`` copies it back only if somebody asks.  float32 / float64 only.
    """
    if isinstance(x, Tensor):
        if x.on_device and (dtype is None or np.dtype(dtype) == x.dtype):
            return Tensor(x, constant=constant, copy=False)
        x = x.data
    arr = np.ascontiguousarray(x, dtype=dtype)
    if arr.dtype not in (np.float32, np.float64):
        raise TypeError(f"device_tensor holds float32 or float64 values, got {arr.dtype}")
    buf = _device.DeviceBuffer(max(arr.nbytes, 16))
    if arr.nbytes:
        buf.upload(arr)
        _device.stats["uploads"] += 1
    return Tensor(_device.DeviceArray(buf, arr.shape, arr.dtype), constant=constant, copy=False)


class Tensor:
    """An N-dimensional array that remembers the operation that produced it."""

    __array_priority__ = 15.0

    def __init__(self, x, *, dtype=None, constant=None, copy=True, ndmin=0, _creator=None, _base=None):
        if constant is not None and not isinstance(constant, bool):
            raise TypeError(f"`constant` must be a boolean value, got: {constant}")
        if not isinstance(ndmin, Integral):
            raise TypeError(f"'{type(ndmin)}' object cannot be interpreted as an integer")
        if isinstance(x, Tensor):
            x = x._value if copy is False else x.data
        self._creator = _creator
        self._guards = []  # weak references to the operations that hold this tensor's value read-only
        if isinstance(x, _device.DeviceArray) and copy is False and not ndmin and (dtype is None or np.dtype(dtype) == x.dtype):
            data = x  # a result that stays on the device until it is read
        elif copy is False:
            data = np.asarray(x, dtype=dtype)
            if ndmin and data.ndim < ndmin:
                data = data[(None,) * (ndmin - data.ndim)]
        else:
            data = np.array(x, dtype=dtype, copy=copy, ndmin=ndmin)
        self._value = data

        kind = data.dtype.type
        is_float = issubclass(kind, np.floating)
        if not is_float and _graph.TRACK_GRAPH:
            if not issubclass(kind, _CONSTANT_ONLY):
                raise TypeError(
                    f"Tensor data must be of an floating type, integer type, or boolean type, received {kind}"
                )
            if constant is False:
                raise ValueError("Integer-valued tensors must be treated as constants.")
        self._constant = (not is_float) if constant is None else constant
        self._grad = None
        self._ops = set()  # weak references to the operations this tensor feeds
        self._base = _base

    # ------------------------------------------------------------------ array-like surface
    @property
    def data(self):
        """The tensor's values as a NumPy array.  The result of an operation stays on the
        device until this is read for the first time (one copy into pinned host memory);
        while the graph that produced or consumes it is alive the array is read-only, like
        every array of a live graph."""
        value = self._value
        if isinstance(value, _device.DeviceArray):
            value = self._to_host()
        return value

    @data.setter
    def data(self, value):
        self._value = value

    def _to_host(self):
        dev = self._value
        arr = dev.host()
        self._value = arr
        holders = [op for op in (ref() for ref in self._guards) if op is not None and op._guarded is not None]
        self._guards = []
        if holders:
            # the graph is alive: the host copy is held read-only like any other array of the
            # graph, which is also what keeps the device buffer a valid copy of it
            _device.attach(arr, dev.buf)
            for op in holders:
                op._guarded.append(_graph.lock(arr))
            _device.drop_pending()
        return arr

    @property
    def on_device(self):
        """True while the values exist on the device only (nothing has read ``data`` yet)."""
        return isinstance(self._value, _device.DeviceArray)

    @property
    def shape(self):
        return self._value.shape

    @property
    def ndim(self):
        return self._value.ndim

    @property
    def size(self):
        return self._value.size

    @property
    def dtype(self):
        return self._value.dtype

    @property
    def constant(self):
        return self._constant

    @property
    def creator(self):
        return self._creator

    @property
    def base(self):
        return self._base

    @property
    def grad(self):
        """The gradient left by the last ``backward()``, as a NumPy array (copied from the
        device on first read) or None."""
        if isinstance(self._grad, _device.DeviceArray):
            self._grad = self._grad.host()
        return self._grad

    def item(self):
        return self.data.item()

    def __array__(self, dtype=None, copy=None):
        if dtype is None:
            return self.data if not copy else self.data.copy()
        return self.data.astype(dtype, copy=bool(copy))

    def __len__(self):
        return len(self.data)

    def __repr__(self):
        return repr(self.data).replace("array", "Tensor").replace("\n", "\n ")

    def null_grad(self):
        self._grad = None
        return self

    # ------------------------------------------------------------------ operators
    # (reference: tensor_base.py:2007-2015, :2378-2384; only what the convolution /
    # pooling chains use, on the device)
    def __mul__(self, other):
        from .math.arithmetic.ops import Multiply

        return self._op(Multiply, self, other)

    def __rmul__(self, other):
        from .math.arithmetic.ops import Multiply

        return self._op(Multiply, other, self)

    def __matmul__(self, other):
        from .math.misc.ops import MatMul

        return self._op(MatMul, self, other)

    def __rmatmul__(self, other):
        from .math.misc.ops import MatMul

        return self._op(MatMul, other, self)

    def sum(self, axis=None, keepdims=False, *, constant=None):
        from .math.sequential.ops import Sum

        return self._op(Sum, self, op_args=(axis, keepdims), constant=constant)

    # ------------------------------------------------------------------ graph construction
    @classmethod
    def _op(cls, Op, *input_vars, op_args=None, op_kwargs=None, constant=None):
        """Run ``Op`` on ``input_vars`` and record it in the graph.

        Non-tensor inputs become constant tensors without a copy; while the
        graph is tracked the input arrays and the result are held read-only
        until the operation is released; the result array is wrapped, not
        copied (reference: tensor_base.py:1086-1212).
        """
        tensor_vars = tuple(
            var if isinstance(var, Tensor) else cls(var, constant=True, copy=False) for var in input_vars
        )
        _device.drop_pending()  # an offer left by an operation that was called directly has lapsed
        guarded = []
        guard = _graph.TRACK_GRAPH and _graph.MEM_GUARD
        if guard:
            guarded = [_graph.lock(a) for a in _graph.arrays_and_bases(tensor_vars)]

        f = Op()
        f._guarded = guarded if guard else None
        try:
            with _device.deferring():  # the result stays on the device until somebody reads it
                op_out = f(*tensor_vars, *(op_args or ()), **(op_kwargs or {}))
        except Exception:
            if guard:
                _graph.release(guarded)
            raise

        if not _graph.TRACK_GRAPH:
            _device.drop_pending()  # the result is handed out writeable: no device copy is kept for it
            return cls(op_out, constant=constant, copy=False)

        for v in input_vars:
            if isinstance(v, Tensor):
                v._grad = None  # a tensor that enters a new graph starts without a gradient

        if constant is None:
            constant = None if any(not v.constant for v in tensor_vars) else True

        ref_f = ReferenceType(f)
        for v in tensor_vars:
            v._ops.add(ref_f)

        out = cls(op_out, constant=constant, copy=False, _creator=f)

        if _graph.MEM_GUARD:
            if not out.on_device:
                guarded.append(_graph.lock(out._value))
            # values that are still on the device have no host array to lock yet: the tensor
            # remembers who holds it, and locks the array on their behalf when it is read
            for t in (*tensor_vars, out):
                if t.on_device:
                    # a device tensor that is never read on the host (a weight in a training loop)
                    # would collect one dead reference per operation: drop them as the list grows
                    if len(t._guards) >= 32:
                        t._guards = [ref for ref in t._guards if ref() is not None]
                    t._guards.append(ref_f)
            finalize(f, _graph.release, guarded)
        _device.drop_pending()
        return out

    # ------------------------------------------------------------------ back-propagation
    def backward(self, grad=None):
        """Back-propagate from this tensor through the graph that produced it,
        leaving ``.grad`` on every non-constant tensor it depends on, then clear
        the graph (reference: tensor_base.py:1294-1340)."""
        if not _graph.TRACK_GRAPH:
            return
        if self.constant:
            self.clear_graph()
            return

        order = deque()
        _collect_and_null(self, set(), order, set())

        if isinstance(grad, Tensor) and grad.on_device:
            grad = grad._value
        if isinstance(grad, _device.DeviceArray) and grad.shape == self.shape and self.dtype in (np.float32, np.float64):
            seed = grad.astype(self.dtype)  # a gradient that is on the device already stays there
        elif grad is not None:
            seed = asarray(grad, dtype=self.dtype)
            if seed.shape != self.shape:
                try:
                    seed = np.multiply(np.ones(self.shape, dtype=self.dtype), seed, dtype=self.dtype)
                    if seed.shape != self.shape:
                        raise ValueError()
                except ValueError:
                    raise ValueError(
                        "`tensor.backward(grad)` was passed a gradient with an incompatible shape.\n"
                        f"`grad` must be broadcast-compatible with `tensor.shape={self.shape}`\n"
                        f"Got `grad.shape={seed.shape}`"
                    )
        elif self._creator is not None and self.on_device and self.size and self.dtype in (np.float16, np.float32, np.float64):
            seed = _device.full(self.shape, self.dtype, 1.0)
        else:
            seed = np.ones(self.shape, dtype=self.dtype)
        self._grad = seed

        try:
            if self._creator is not None:
                for t in order:
                    t._backward()
        finally:
            _device.drop_transients()
        self.clear_graph()

    def _backward(self):
        assert self._grad is not None, f"backprop was triggered on a tensor with no gradient\n{self}"
        assert self._grad.shape == self.shape, (
            "A tensor and its associated gradient must possess the same shape. Got:"
            f"\ntensor-shape: {self.shape}\ngrad-shape: {self._grad.shape}"
        )
        if self._creator is not None:
            grad = self._grad if self._creator.takes_device_arrays else self.grad
            with _device.deferring():
                self._creator.backward(grad)

    def clear_graph(self):
        """Detach this tensor and everything upstream of it from the graph; the
        operations are dropped, which releases the read-only hold on their arrays
        (reference: tensor_base.py:1461-1498)."""
        self._ops.clear()
        if self._creator is None:
            return
        creator = self._creator
        self._creator = None
        for var in creator.variables:
            var.clear_graph()


def _collect_and_null(t, seen, order, on_path):
    """Depth-first topological sort from the terminal tensor towards the leaves,
    nulling every gradient on the way (reference: mygrad/_utils/__init__.py:36-73)."""
    t._grad = None
    if t.constant or id(t) in seen:
        return
    assert id(t) not in on_path, "Computational graph contains a cycle"
    on_path.add(id(t))
    if t.creator is not None:
        for parent in t.creator.variables:
            _collect_and_null(parent, seen, order, on_path)
    on_path.discard(id(t))
    seen.add(id(t))
    order.appendleft(t)
