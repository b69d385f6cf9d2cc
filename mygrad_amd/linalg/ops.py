"""``EinSum`` on the MI355X (reference: ``mygrad/linalg/ops.py:79-262``).

An Einstein summation of one or two operands is brought into the form the matrix-product
kernels take: labels that occur in one operand only and not in the result are summed away
first (``mg_sum_over``); the others fall into batch labels (both operands and the result),
contracted labels (both operands, not the result), row labels (first operand and result)
and column labels (second operand and result); the operands are transposed on the device
to ``(batch, rows, contracted)`` and ``(batch, contracted, columns)`` (``mg_permute``),
multiplied (``mg_matmul``, one launch per batch entry), and the product is transposed into
the order the subscripts ask for.  The gradient of an operand is, as in the reference, the
same kind of summation with the incoming gradient in the operand's place.

What runs: one or two float32 / float64 operands, no label repeated within one operand (no
traces or diagonals), every label of the same length wherever it occurs.  Anything else
raises ``NotImplementedError``; there is no CPU fallback.  The result is always a new
array, never a view of an operand."""

from collections import Counter
from itertools import chain

import numpy as np

from .. import _device, _hip, _reduce
from ..errors import SkipGradient
from ..operation_base import Operation

__all__ = ["EinSum"]


def _prod(values):
    total = 1
    for v in values:
        total *= int(v)
    return total


def _sum_away(buf, lbls, gone, sizes, dtype):
    """``buf`` with the labels in ``gone`` summed over -> (buffer, remaining labels)."""
    axes = tuple(i for i, lbl in enumerate(lbls) if lbl in gone)
    if not axes:
        return buf, lbls
    shape = tuple(sizes[lbl] for lbl in lbls)
    return _reduce.sum_axes(buf, shape, axes, dtype), "".join(lbl for lbl in lbls if lbl not in gone)


def _ordered(buf, lbls, order, sizes, dtype):
    """``buf`` (axes ``lbls``) transposed so that its axes are ``order``."""
    perm = tuple(lbls.index(lbl) for lbl in order)
    return _reduce.permute(buf, tuple(sizes[lbl] for lbl in lbls), perm, dtype)


def contract(operands, out_lbls, sizes, dtype):
    """Device buffer with ``einsum(operands -> out_lbls)``: ``operands`` is one or two pairs
    (device buffer, labels), ``sizes`` maps each label to its length (none of them zero)."""
    lib, code, item = _hip.lib(), _hip.dtype_code(dtype), dtype.itemsize
    if len(operands) == 1:
        (buf, lbls), = operands
        buf, lbls = _sum_away(buf, lbls, set(lbls) - set(out_lbls), sizes, dtype)
        return _ordered(buf, lbls, out_lbls, sizes, dtype)
    (abuf, albl), (bbuf, blbl) = operands
    abuf, albl = _sum_away(abuf, albl, set(albl) - set(blbl) - set(out_lbls), sizes, dtype)
    bbuf, blbl = _sum_away(bbuf, blbl, set(blbl) - set(albl) - set(out_lbls), sizes, dtype)
    batch = "".join(lbl for lbl in out_lbls if lbl in albl and lbl in blbl)
    summed = "".join(lbl for lbl in albl if lbl in blbl and lbl not in out_lbls)
    rows = "".join(lbl for lbl in out_lbls if lbl in albl and lbl not in blbl)
    cols = "".join(lbl for lbl in out_lbls if lbl in blbl and lbl not in albl)
    abuf = _ordered(abuf, albl, batch + rows + summed, sizes, dtype)
    bbuf = _ordered(bbuf, blbl, batch + summed + cols, sizes, dtype)
    B, M, K, N = (_prod(sizes[lbl] for lbl in group) for group in (batch, rows, summed, cols))
    out = _device.DeviceBuffer(max(B * M * N * item, 16))
    for b in range(B):
        _hip.check(lib.mg_matmul(code, 1, M, K, N, abuf.ptr + b * M * K * item, bbuf.ptr + b * K * N * item, out.ptr + b * M * N * item))
    return _ordered(out, batch + rows + cols, out_lbls, sizes, dtype)


class EinSum(Operation):
    gradient_on_device = True

    def __call__(self, *variables, in_lbls, out_lbls, out=None, optimize=False):
        self.in_lbls = in_lbls.split(",")
        self.out_lbls = out_lbls
        self.variables = variables
        self.optimize = optimize
        self._cache = None  # how often each (tensor, labels) pair occurs; see backward_var
        if out is not None:
            raise NotImplementedError("einsum on the GPU does not write into an existing array (out=...)")
        arrays = [v.data for v in variables]

        # the checks np.einsum makes, with its exception type
        if len(self.in_lbls) != len(arrays):
            raise ValueError("more operands provided to einstein sum function than specified in the subscripts string"
                             if len(arrays) > len(self.in_lbls) else
                             "fewer operands provided to einstein sum function than specified in the subscripts string")
        sizes = {}
        for lbls, arr in zip(self.in_lbls, arrays):
            if len(lbls) != arr.ndim:
                raise ValueError(f"einstein sum subscripts string '{lbls}' does not match the {arr.ndim} axes of its operand")
            for lbl, n in zip(lbls, arr.shape):
                if sizes.setdefault(lbl, n) != n:
                    if 1 in (sizes[lbl], n):
                        raise NotImplementedError(f"einsum on the GPU does not broadcast label '{lbl}' (lengths {sizes[lbl]} and {n})")
                    raise ValueError(f"operands could not be broadcast together: label '{lbl}' has lengths {sizes[lbl]} and {n}")
        if len(set(out_lbls)) != len(out_lbls):
            raise ValueError(f"einstein sum subscripts string includes output subscript more than once: '{out_lbls}'")
        if not set(out_lbls) <= set(sizes):
            raise ValueError(f"einstein sum subscripts string included output subscript which never appeared in an input: '{out_lbls}'")

        if len(arrays) not in (1, 2):
            raise NotImplementedError(f"einsum on the GPU takes one or two operands, got {len(arrays)} (no CPU fallback)")
        if any(len(set(lbls)) != len(lbls) for lbls in self.in_lbls):
            raise NotImplementedError("einsum on the GPU does not take a label twice within one operand (traces, diagonals)")
        dtype = np.dtype(np.result_type(*arrays))
        if dtype not in (np.float32, np.float64):
            raise TypeError(f"einsum runs on the GPU in float32 or float64, got {[str(a.dtype) for a in arrays]} (there is no CPU fallback)")
        self._dtype, self._sizes = dtype, sizes

        out_shape = tuple(sizes[lbl] for lbl in out_lbls)
        if 0 in sizes.values():  # an empty sum is zero, an empty result has nothing in it
            return np.zeros(out_shape, dtype=dtype)
        operands = [(_device.to_device(arr, dtype), lbls) for arr, lbls in zip(arrays, self.in_lbls)]
        ob = contract(operands, out_lbls, sizes, dtype)
        if any(ob is buf for buf, _ in operands):  # nothing was summed or moved: the result is a copy
            copy = _device.DeviceBuffer(max(_prod(out_shape) * dtype.itemsize, 16))
            _hip.check(_hip.lib().mg_memcpy_d2d(copy.ptr, ob.ptr, _prod(out_shape) * dtype.itemsize))
            ob = copy
        result = _device.download(ob, out_shape, dtype)
        _device.attach(result, ob)
        return result

    @property
    def cache(self):
        # built on first use, as in the reference (linalg/ops.py:112-122): the count of each
        # (tensor, labels) pair among the operands; one gradient is computed per distinct pair
        if self._cache is None:
            self._cache = Counter(zip((id(v) for v in self.variables), self.in_lbls))
        return self._cache

    def backward_var(self, grad, index, **kwargs):
        """forward ``"ijk,k->ji", x, y``: the gradient of x is ``"ji,k->ijk", grad, y`` and that of
        y is ``"ji,ijk->k", grad, x`` (linalg/ops.py:124-218)."""
        others = list(self.in_lbls)
        var_lbl = others.pop(index)
        var = self.variables[index]
        factor = self.cache[(id(var), var_lbl)]
        if factor == 0:  # this (tensor, labels) pair has had its gradient, scaled by its count
            raise SkipGradient()
        self.cache[(id(var), var_lbl)] = 0
        dtype, sizes = self._dtype, self._sizes
        if var.data.size == 0:
            return np.zeros(var.shape, dtype=dtype)
        if 0 in sizes.values():
            return np.zeros(var.shape, dtype=dtype)

        # labels of this operand that were summed away on their own occur nowhere else: the
        # gradient is the same along them (linalg/ops.py:170-190)
        elsewhere = set(chain.from_iterable(others)) | set(self.out_lbls)
        found = "".join(lbl for lbl in var_lbl if lbl in elsewhere)
        operands = [(_device.to_device(np.ascontiguousarray(grad), dtype), self.out_lbls)]
        operands += [(_device.to_device(v.data, dtype), lbls)
                     for n, (v, lbls) in enumerate(zip(self.variables, self.in_lbls)) if n != index]
        ob = contract(operands, found, sizes, dtype)
        if found != var_lbl:
            ob = _reduce.broadcast(ob, tuple(sizes[lbl] if lbl in elsewhere else 1 for lbl in var_lbl), var.shape, dtype)
        nbytes = var.data.size * dtype.itemsize
        if factor > 1 or any(ob is buf for buf, _ in operands):
            # a buffer of its own, scaled by the number of times the pair occurs
            scale = _device.to_device(np.array(float(factor), dtype=dtype))
            ones = _device.DeviceBuffer(max(nbytes, 16))
            _hip.check(_hip.lib().mg_fill_from(_hip.dtype_code(dtype), var.data.size, scale.ptr, ones.ptr))
            scaled = _device.DeviceBuffer(max(nbytes, 16))
            _hip.check(_hip.lib().mg_multiply(_hip.dtype_code(dtype), var.data.size, ob.ptr, ones.ptr, scaled.ptr))
            ob = scaled
        out = _device.download(ob, var.shape, dtype)
        _device.attach_transient(out, ob)
        return out
