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

__all__ = ["Tensor", "tensor", "asarray"]

_CONSTANT_ONLY = (np.integer, np.bool_)


def asarray(a, dtype=None):
    """``numpy.asarray`` that unwraps tensors."""
    if isinstance(a, Tensor):
        a = a.data
    return np.asarray(a, dtype=dtype)


def tensor(x, *, dtype=None, constant=None, copy=True, ndmin=0):
    """Create a tensor (counterpart of ``mygrad.tensor``)."""
    return Tensor(x, dtype=dtype, constant=constant, copy=copy, ndmin=ndmin)


class Tensor:
    """An N-dimensional array that remembers the operation that produced it."""

    __array_priority__ = 15.0

    def __init__(self, x, *, dtype=None, constant=None, copy=True, ndmin=0, _creator=None, _base=None):
        if constant is not None and not isinstance(constant, bool):
            raise TypeError(f"`constant` must be a boolean value, got: {constant}")
        if not isinstance(ndmin, Integral):
            raise TypeError(f"'{type(ndmin)}' object cannot be interpreted as an integer")
        if isinstance(x, Tensor):
            x = x.data
        self._creator = _creator
        if copy is False:
            data = np.asarray(x, dtype=dtype)
            if ndmin and data.ndim < ndmin:
                data = data[(None,) * (ndmin - data.ndim)]
        else:
            data = np.array(x, dtype=dtype, copy=copy, ndmin=ndmin)
        self.data = data

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
    def shape(self):
        return self.data.shape

    @property
    def ndim(self):
        return self.data.ndim

    @property
    def size(self):
        return self.data.size

    @property
    def dtype(self):
        return self.data.dtype

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
        guarded = []
        guard = _graph.TRACK_GRAPH and _graph.MEM_GUARD
        if guard:
            guarded = [_graph.lock(a) for a in _graph.arrays_and_bases(tensor_vars)]

        f = Op()
        try:
            op_out = f(*tensor_vars, *(op_args or ()), **(op_kwargs or {}))
        except Exception:
            if guard:
                _graph.release(guarded)
            raise

        if not _graph.TRACK_GRAPH:
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
            guarded.append(_graph.lock(out.data))
            finalize(f, _graph.release, guarded)
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

        if grad is not None:
            seed = asarray(grad, dtype=self.dtype)
            if seed.shape != self.shape:
                try:
                    seed = np.multiply(np.full_like(self.data, fill_value=1.0), seed, dtype=self.dtype)
                    if seed.shape != self.shape:
                        raise ValueError()
                except ValueError:
                    raise ValueError(
                        "`tensor.backward(grad)` was passed a gradient with an incompatible shape.\n"
                        f"`grad` must be broadcast-compatible with `tensor.shape={self.shape}`\n"
                        f"Got `grad.shape={seed.shape}`"
                    )
        else:
            seed = np.full_like(self.data, fill_value=1.0)
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
            self._creator.backward(self._grad)

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
