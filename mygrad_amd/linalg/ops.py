"""``EinSum`` on the MI355X (reference: ``mygrad/linalg/ops.py:79-262``).

An Einstein summation (of one or two operands at a time) is brought into the form the matrix-product
kernels take: labels that occur in one operand only and not in the result are summed away
first (``mg_sum_over``); the others fall into batch labels (both operands and the result),
contracted labels (both operands, not the result), row labels (first operand and result)
and column labels (second operand and result); the operands are transposed on the device
to ``(batch, rows, contracted)`` and ``(batch, contracted, columns)`` (``mg_permute``),
multiplied (``mg_matmul_batched`` for a stack of small products, else ``mg_matmul`` with one
launch per batch entry), and the product is transposed into
the order the subscripts ask for.  Two arrangements need no transposition of the large
tensors and are recognised first: a convolution with a one-element window written as a
summation (``"nchw,fc->nfhw"`` and its input gradient: ``mg_matmul`` with the leading labels
as the batch) and its filter gradient (``"nfhw,nchw->fc"``: ``mg_matmul_da``); a plain
matrix product is the first of them.  The gradient of an operand is, as in the reference,
the same kind of summation with the incoming gradient in the operand's place.

What runs: float32 / float64 operands (more than two are contracted pairwise from the
left); a label repeated within one operand is taken along its diagonal first
(``mg_strided_copy``), and its gradient is written back along that diagonal into zeros; an
axis of length one under a label that is longer elsewhere is broadcast (a diagonal of
length one included); ``out=`` names a NumPy array that receives the result.  Anything else
raises ``NotImplementedError``; there is no CPU fallback.  Without ``out`` the result is a
new array, never a view of an operand."""

from collections import Counter
from itertools import chain

import numpy as np

from .. import _device, _hip, _reduce
from ..errors import SkipGradient
from ..math.misc.ops import SMALL_PAIR_FLOPS
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


def _block(lbls, members):
    """Where the labels ``members`` sit in ``lbls`` if they form one run there: (start, stop),
    (n, n) for no members at all; None if they are scattered."""
    at = [n for n, lbl in enumerate(lbls) if lbl in members]
    if not at:
        return len(lbls), len(lbls)
    return (at[0], at[-1] + 1) if at == list(range(at[0], at[-1] + 1)) else None


def _shared_filter_form(operands, out_lbls, sizes, dtype):
    """``out[o, m, i] = sum_k a[m, k] x[o, k, i]`` without moving ``x`` or the result: one operand
    (``x``) already has its contracted labels in one run with free labels before (``o``) and
    after (``i``) it, and the result is those with the other operand's free labels (``m``) in
    between -- a convolution with a one-element window read straight from its tensors
    (``mg_matmul`` with ``o`` as the batch).  Only the other operand is re-ordered."""
    lib, code, item = _hip.lib(), _hip.dtype_code(dtype), dtype.itemsize
    for which in sorted((0, 1), key=lambda n: -_prod(sizes[lbl] for lbl in operands[n][1])):  # the larger one as x
        (xbuf, xl), (abuf, al) = operands[which], operands[1 - which]
        summed = [lbl for lbl in xl if lbl in al]
        if not summed or any(lbl in out_lbls for lbl in summed):
            continue
        run = _block(xl, summed)
        if run is None:
            continue
        outer, inner = xl[: run[0]], xl[run[1] :]
        rows = "".join(lbl for lbl in out_lbls if lbl in al)
        if out_lbls != outer + rows + inner:
            continue
        abuf = _ordered(abuf, al, rows + xl[run[0] : run[1]], sizes, dtype)
        B, M, K, N = (_prod(sizes[lbl] for lbl in group) for group in (outer, rows, summed, inner))
        out = _device.DeviceBuffer(max(B * M * N * item, 16))
        _hip.check(lib.mg_matmul(code, B, M, K, N, abuf.ptr, xbuf.ptr, out.ptr))
        return out
    return None


def _joint_sum_form(operands, out_lbls, sizes, dtype):
    """``out[r, c] = sum_{o, i} g[o, r, i] x[o, c, i]``: both operands carry the contracted labels
    as the same run before and the same run after their own free labels -- the filter gradient
    of that convolution (``mg_matmul_da`` with ``o`` as the batch).  Neither operand moves; the
    (small) result is put into the order asked for."""
    lib, code, item = _hip.lib(), _hip.dtype_code(dtype), dtype.itemsize
    (gbuf, gl), (xbuf, xl) = operands
    summed = set(gl) & set(xl)
    if not summed or summed & set(out_lbls):
        return None
    grun, xrun = _block(gl, set(gl) - summed), _block(xl, set(xl) - summed)
    if grun is None or xrun is None:
        return None
    if gl[: grun[0]] != xl[: xrun[0]] or gl[grun[1] :] != xl[xrun[1] :]:
        return None
    outer, inner = gl[: grun[0]], gl[grun[1] :]
    rows, cols = gl[grun[0] : grun[1]], xl[xrun[0] : xrun[1]]
    B, M, K, N = (_prod(sizes[lbl] for lbl in group) for group in (outer, rows, cols, inner))
    out = _device.DeviceBuffer(max(M * K * item, 16))
    _hip.check(lib.mg_matmul_da(code, B, M, K, N, gbuf.ptr, xbuf.ptr, out.ptr))
    return _ordered(out, rows + cols, out_lbls, sizes, dtype)


def _last_of_each(lbls):
    """``lbls`` with every label kept once, at its last position: "ijikik" -> "jik"
    (the order the reference reduces a repeated label to, linalg/ops.py:21-42)."""
    return "".join(lbl for n, lbl in enumerate(lbls) if lbl not in lbls[n + 1 :])


def _diagonal_strides(lbls, once, sizes):
    """Element strides that walk the C-contiguous operand labelled ``lbls`` along ``once``:
    a label that occurs several times moves along all of its axes together."""
    strides, step = {}, 1
    for lbl in reversed(lbls):
        strides[lbl] = strides.get(lbl, 0) + step
        step *= sizes[lbl]
    return [strides[lbl] for lbl in once]


def _strided(buf, lbls, once, sizes, dtype, scatter):
    """gather: the operand ``buf`` (labels ``lbls``, some repeated) -> its diagonal array labelled
    ``once``.  scatter: the array ``buf`` labelled ``once`` -> zeros of the operand's shape with
    ``buf`` written along those diagonals."""
    import ctypes

    lib, item = _hip.lib(), dtype.itemsize
    full = _prod(sizes[lbl] for lbl in lbls)
    dense = _prod(sizes[lbl] for lbl in once)
    shape = (ctypes.c_int64 * len(once))(*(sizes[lbl] for lbl in once))
    strides = (ctypes.c_int64 * len(once))(*_diagonal_strides(lbls, once, sizes))
    out = _device.DeviceBuffer(max((full if scatter else dense) * item, 16))
    if scatter:
        _hip.check(lib.mg_memset_zero(out.ptr, full * item))
    _hip.check(lib.mg_strided_copy(item, len(once), shape, strides, full, int(scatter), buf.ptr, out.ptr))
    return out


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
    operands = [(abuf, albl), (bbuf, blbl)]

    # the two forms that leave the large tensors where they are
    long_sum = _prod(sizes[lbl] for lbl in set(albl) & set(blbl)) >= _prod(sizes[lbl] for lbl in out_lbls)
    forms = (_joint_sum_form, _shared_filter_form) if long_sum else (_shared_filter_form, _joint_sum_form)
    for form in forms:
        out = form(operands, out_lbls, sizes, dtype)
        if out is not None:
            return out

    # the general way: both operands transposed to (batch, free, summed) order
    batch = "".join(lbl for lbl in out_lbls if lbl in albl and lbl in blbl)
    summed = "".join(lbl for lbl in albl if lbl in blbl and lbl not in out_lbls)
    rows = "".join(lbl for lbl in out_lbls if lbl in albl and lbl not in blbl)
    cols = "".join(lbl for lbl in out_lbls if lbl in blbl and lbl not in albl)
    B, M, K, N = (_prod(sizes[lbl] for lbl in group) for group in (batch, rows, summed, cols))
    out = _device.DeviceBuffer(max(B * M * N * item, 16))
    if B > 1 and 2 * M * K * N <= SMALL_PAIR_FLOPS:
        # many small products: one launch for all of them; an operand that already lies
        # transposed is read that way instead of being moved
        trans_a = albl == batch + summed + rows and M > 1 and K > 1
        trans_b = blbl == batch + cols + summed and N > 1 and K > 1
        if not trans_a:
            abuf = _ordered(abuf, albl, batch + rows + summed, sizes, dtype)
        if not trans_b:
            bbuf = _ordered(bbuf, blbl, batch + summed + cols, sizes, dtype)
        _hip.check(lib.mg_matmul_batched(code, B, M, K, N, int(trans_a), int(trans_b), abuf.ptr, bbuf.ptr, out.ptr))
        return _ordered(out, batch + rows + cols, out_lbls, sizes, dtype)
    if K >= 4 * max(M, N):
        # a long sum and a small result: the filter-gradient kernels, out = a @ b^T over the long axis
        abuf = _ordered(abuf, albl, batch + rows + summed, sizes, dtype)
        bbuf = _ordered(bbuf, blbl, batch + cols + summed, sizes, dtype)
        for b in range(B):
            _hip.check(lib.mg_matmul_da(code, 1, M, N, K, abuf.ptr + b * M * K * item, bbuf.ptr + b * N * K * item,
                                        out.ptr + b * M * N * item))
        return _ordered(out, batch + rows + cols, out_lbls, sizes, dtype)
    if N < M:  # the longer free axis plays the positions of the convolution, the other its filters
        (abuf, albl, rows, M), (bbuf, blbl, cols, N) = (bbuf, blbl, cols, N), (abuf, albl, rows, M)
    abuf = _ordered(abuf, albl, batch + rows + summed, sizes, dtype)
    bbuf = _ordered(bbuf, blbl, batch + summed + cols, sizes, dtype)
    for b in range(B):
        _hip.check(lib.mg_matmul(code, 1, M, K, N, abuf.ptr + b * M * K * item, bbuf.ptr + b * K * N * item, out.ptr + b * M * N * item))
    return _ordered(out, batch + rows + cols, out_lbls, sizes, dtype)


def contract_all(operands, out_lbls, sizes, dtype):
    """``contract`` for any number of operands: the first two are contracted onto the labels
    that are still needed (by the operands that follow, or by the result) until two are left."""
    operands = list(operands)
    while len(operands) > 2:
        (abuf, albl), (bbuf, blbl) = operands[:2]
        needed = set(out_lbls) | set(chain.from_iterable(lbls for _, lbls in operands[2:]))
        keep = "".join(dict.fromkeys(lbl for lbl in albl + blbl if lbl in needed))
        operands[:2] = [(contract([(abuf, albl), (bbuf, blbl)], keep, sizes, dtype), keep)]
    return contract(operands, out_lbls, sizes, dtype)


class EinSum(Operation):
    takes_device_arrays = True

    gradient_on_device = True

    def __call__(self, *variables, in_lbls, out_lbls, out=None, optimize=False):
        self.in_lbls = in_lbls.split(",")
        self.out_lbls = out_lbls
        self.variables = variables
        self.optimize = optimize
        self._cache = None  # how often each (tensor, labels) pair occurs; see backward_var
        if out is not None and not isinstance(out, np.ndarray):
            raise TypeError("keyword parameter out must be an array for einsum")
        arrays = [_device.value_of(v) for v in variables]

        # the checks np.einsum makes, with its exception type
        if len(self.in_lbls) != len(arrays):
            raise ValueError("more operands provided to einstein sum function than specified in the subscripts string"
                             if len(arrays) > len(self.in_lbls) else
                             "fewer operands provided to einstein sum function than specified in the subscripts string")
        sizes = {}
        for nth, (lbls, arr) in enumerate(zip(self.in_lbls, arrays)):
            if len(lbls) != arr.ndim:
                raise ValueError(f"einstein sum subscripts string '{lbls}' does not match the {arr.ndim} axes of its operand")
            own = {}  # a label repeated within the operand walks a diagonal: its axes must agree
            for lbl, n in zip(lbls, arr.shape):
                if own.setdefault(lbl, n) != n:
                    raise ValueError(f"dimensions in operand {nth} for collapsing index '{lbl}' "
                                     f"don't match ({own[lbl]} != {n})")
                have = sizes.get(lbl)
                if have is None or have == 1:
                    sizes[lbl] = n
                elif n not in (1, have):
                    raise ValueError(f"operands could not be broadcast together: label '{lbl}' has lengths {have} and {n}")
        # An axis of length one under a label that is longer elsewhere is broadcast: the operand
        # does not depend on that label, so the label is struck from it (same memory), and
        # its gradient is summed over the label like over any label it does not carry.  A label
        # repeated within the operand goes or stays with all of its axes (they agree in length).
        self._lbls = ["".join(lbl for lbl, n in zip(lbls, arr.shape) if n == sizes[lbl])
                      for lbls, arr in zip(self.in_lbls, arrays)]
        if len(set(out_lbls)) != len(out_lbls):
            raise ValueError(f"einstein sum subscripts string includes output subscript more than once: '{out_lbls}'")
        if not set(out_lbls) <= set(sizes):
            raise ValueError(f"einstein sum subscripts string included output subscript which never appeared in an input: '{out_lbls}'")

        if any(len(lbls) - len(set(lbls)) > 0 and len(set(lbls)) > 6 for lbls in self._lbls):
            raise NotImplementedError("einsum on the GPU walks diagonals of operands with at most six distinct labels")
        dtype = np.dtype(np.result_type(*(a.dtype for a in arrays)))
        if dtype not in (np.float32, np.float64):
            raise TypeError(f"einsum runs on the GPU in float32 or float64, got {[str(a.dtype) for a in arrays]} (there is no CPU fallback)")
        self._dtype, self._sizes = dtype, sizes

        out_shape = tuple(sizes[lbl] for lbl in out_lbls)
        if out is not None:
            # the checks np.einsum makes of its target, before anything is computed
            if out.ndim != len(out_shape):
                raise ValueError(f"out parameter does not have the correct number of dimensions, has {out.ndim} but should have {len(out_shape)}")
            if out.shape != out_shape:
                raise ValueError(f"operands could not be broadcast together: out has shape {out.shape}, the result {out_shape}")
            if not out.flags.writeable:
                raise ValueError("operand array with iterator write flag set is read-only")
            if not np.can_cast(dtype, out.dtype, "safe"):
                raise TypeError(f"Iterator requested dtype could not be cast from {dtype!r} to {out.dtype!r}, the operand {len(arrays)} dtype, "
                                "according to the rule 'safe'")
        if 0 in sizes.values():  # an empty sum is zero, an empty result has nothing in it
            if out is not None:
                out[...] = 0
                return out
            return np.zeros(out_shape, dtype=dtype)
        operands = [self._operand(arr, lbls) for arr, lbls in zip(arrays, self._lbls)]
        ob = contract_all(operands, out_lbls, sizes, dtype)
        if any(ob is buf for buf, _ in operands):  # nothing was summed or moved: the result is a copy
            copy = _device.DeviceBuffer(max(_prod(out_shape) * dtype.itemsize, 16))
            _hip.check(_hip.lib().mg_memcpy_d2d(copy.ptr, ob.ptr, _prod(out_shape) * dtype.itemsize))
            ob = copy
        if out is not None:
            # the values cross to the host now, into the caller's array (which may be strided or
            # of a wider type); the buffer stays its device copy when the two hold the same bytes
            if out.dtype == dtype and out.flags["C_CONTIGUOUS"]:
                ob.download_into(out)
                _device.attach(out, ob)
            else:
                np.copyto(out, _device.download(ob, out_shape, dtype, now=True), casting="safe")
            return out
        result = _device.download(ob, out_shape, dtype)
        _device.attach(result, ob)
        return result

    def _operand(self, arr, lbls):
        """(device buffer, labels) of one operand; a label that occurs twice is taken along its
        diagonal first, which leaves every label once."""
        buf = _device.to_device(arr, self._dtype)
        once = _last_of_each(lbls)
        if once == lbls:
            return buf, lbls
        return _strided(buf, lbls, once, self._sizes, self._dtype, scatter=False), once

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
        var = self.variables[index]
        pair = (id(var), self.in_lbls[index])
        factor = self.cache[pair]
        if factor == 0:  # this (tensor, labels) pair has had its gradient, scaled by its count
            raise SkipGradient()
        self.cache[pair] = 0
        others = list(self._lbls)  # labels with broadcast axes struck
        var_lbl = others.pop(index)
        dtype, sizes = self._dtype, self._sizes
        if _device.value_of(var).size == 0:
            return np.zeros(var.shape, dtype=dtype)
        if 0 in sizes.values():
            return np.zeros(var.shape, dtype=dtype)

        # labels of this operand that were summed away on their own occur nowhere else: the
        # gradient is the same along them (linalg/ops.py:170-190)
        elsewhere = set(chain.from_iterable(others)) | set(self.out_lbls)
        once = _last_of_each(var_lbl)  # the operand's labels with its diagonals taken (linalg/ops.py:147-163)
        found = "".join(lbl for lbl in once if lbl in elsewhere)
        operands = [(_device.to_device(grad if isinstance(grad, _device.DeviceArray) else np.ascontiguousarray(grad), dtype), self.out_lbls)]
        operands += [self._operand(_device.value_of(v), lbls) for n, (v, lbls) in enumerate(zip(self.variables, self._lbls)) if n != index]
        ob = contract_all(operands, found, sizes, dtype)
        if found != once:
            ob = _reduce.broadcast(ob, tuple(sizes[lbl] if lbl in elsewhere else 1 for lbl in once),
                                   tuple(sizes[lbl] for lbl in once), dtype)
        if once != var_lbl:
            # the gradient lives on the diagonals the forward pass read; everything off them is
            # zero (the reference writes through a strided view of zeros, linalg/ops.py:220-262)
            ob = _strided(ob, var_lbl, once, sizes, dtype, scatter=True)
        nbytes = _device.value_of(var).size * dtype.itemsize
        if factor > 1 or any(ob is buf for buf, _ in operands):
            # a buffer of its own, scaled by the number of times the pair occurs
            ones = _device.DeviceBuffer(max(nbytes, 16))
            _hip.check(_hip.lib().mg_fill_value(_hip.dtype_code(dtype), _device.value_of(var).size, float(factor), ones.ptr))
            scaled = _device.DeviceBuffer(max(nbytes, 16))
            _hip.check(_hip.lib().mg_multiply(_hip.dtype_code(dtype), _device.value_of(var).size, ob.ptr, ones.ptr, scaled.ptr))
            ob = scaled
        out = _device.download(ob, var.shape, dtype)
        _device.attach_transient(out, ob)
        return out
