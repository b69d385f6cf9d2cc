"""NumPy restatement of the reference conv_nd / max_pool algorithm.

TEST INFRASTRUCTURE: this module is the checker (and the timed CPU baseline of
the benchmark); the shipped package never imports it.

Every function follows the reference implementation named in its docstring
(paths relative to the reference checkout) and hands the bulk arithmetic to the
same NumPy routines the reference uses, so that on one NumPy/BLAS build it
produces the reference's numbers: bit-for-bit for pooling, and up to BLAS
summation order for convolution.

``validate=False`` switches off the exact-integer output-shape check of the
Operation layer, leaving the flooring placement rule of the window helper; the
benchmark shapes that the reference's validation rejects are checked that way.

Pinning (what holds each function to the reference without importing it):

  window_view      definition ``out[g] == arr[..., g*S : g*S + W*D : D]`` on
                   random cases + the reference's docstring / memory vectors
  conv_forward     reference known answers (1-D, 2-D, triangle response,
                   padding-only image), brute-force loops
  conv_backward_x  reference docstring gradient, brute-force loops,
  conv_backward_w  adjoint identity <conv(x,w),g> = <x,dx> = <w,dw>,
                   central differences
  pool_forward     three reference known-answer cases + the docstring case
  pool_backward    with a tie, brute-force loops on tie-heavy integer inputs
  pool_argmax      the docstring tie case read as offsets, first-NaN case, loops
  relu_forward     the reference's docstring vectors (``-0.0`` for negative inputs,
  relu_backward    gradient ``[0, 0, 0, 1, 1]``); one IEEE multiply per element
  multiply, multiply_backward, sum_all, sum_all_backward
                   single calls of the NumPy routine the reference calls
                   (``np.multiply``, ``np.sum``, ``np.full``); ``sum_all`` is
                   additionally held to ``math.fsum`` and closed forms in the tests
  einsum_forward   ``np.einsum`` itself, held to the reference's docstring vectors
  einsum_backward  central differences, the adjoint identity <einsum(a, b), g> =
                   <a, grad_a> = <b, grad_b>, loops over every index
  sum_axes, sum_axes_backward, reduce_broadcast, multiply_broadcast_backward
                   ``np.sum`` itself, held to ``math.fsum`` per kept entry and to loops;
                   the two gradients to loops over every index and to the adjoint
                   identities <sum(x), g> = <x, backward(g)> and
                   <a * b, g> = <a, grad_a> = <b, grad_b>
  batchnorm_forward
                   the reference's docstring vector; its tests' second formulation
                   (mean / variance / division composed of primitives); closed forms
                   (per-channel mean of the output is ``beta``, its variance
                   ``gamma**2 * var / (var + eps)``)
  batchnorm_backward
                   central differences of ``sum(grad * batchnorm(x))`` in x, gamma
                   and beta; the invariants ``sum_c(dx) == 0`` and, at ``eps == 0``,
                   ``sum_c(dx * x_norm) == 0``
  matmul_forward   a single call of ``np.matmul`` (what the reference's ufunc calls); the
                   reference's docstring vectors; triple loops on small operands
  matmul_backward  triple loops; the adjoint identities
                   ``<a @ b, g> == <a, da> == <b, db>`` (the product is linear in each)
  repeat_forward   a single call of ``np.repeat`` (what the reference calls); the
                   reference's four docstring vectors
  repeat_backward  element-by-element loops; the adjoint identity
                   ``<repeat(a), g> == <a, repeat_backward(g)>`` (repeat is linear)
"""

from numbers import Integral

import numpy as np
from numpy.lib.stride_tricks import as_strided

__all__ = [
    "window_view",
    "normalize_conv_args",
    "conv_out_shape",
    "conv_forward",
    "conv_backward_x",
    "conv_backward_w",
    "multiply",
    "multiply_backward",
    "relu_forward",
    "relu_backward",
    "sum_all",
    "sum_all_backward",
    "batchnorm_forward",
    "batchnorm_backward",
    "repeat_forward",
    "repeat_backward",
    "matmul_forward",
    "matmul_backward",
    "pool_out_shape",
    "sum_axes",
    "sum_axes_backward",
    "reduce_broadcast",
    "multiply_broadcast_backward",
    "einsum_forward",
    "einsum_backward",
    "pool_forward",
    "pool_argmax",
    "pool_backward",
]


# --------------------------------------------------------------------------- #
# window helper
# --------------------------------------------------------------------------- #
def window_view(arr, window_shape, step, dilation=None):
    """Read-only strided window view, shape ``(G..., lead..., W...)``.

    Follows src/mygrad/nnet/layers/utils.py:123-228 (validation :123-196,
    stride arithmetic :198-228).  ``view[g, lead, w] = arr[lead, g*S + w*D]``
    with ``G = (x - ((W-1)*D + 1)) // S + 1`` (floor).
    """
    if not hasattr(window_shape, "__iter__"):
        raise TypeError(f"`window_shape` must be a sequence of positive integers, got: {window_shape}")
    window_shape = tuple(window_shape)
    if any(not isinstance(w, Integral) or w <= 0 for w in window_shape):
        raise TypeError(f"`window_shape` must be a sequence of positive integers, got: {window_shape}")
    m = len(window_shape)
    if m > arr.ndim:
        raise ValueError(
            f"`window_shape` ({window_shape}) cannot specify more values than `arr.ndim` ({arr.ndim})."
        )

    if isinstance(step, Integral):
        step = (int(step),) * m
    elif hasattr(step, "__iter__"):
        step = tuple(step)
    else:
        raise TypeError(f"`step` must be a positive integer or a sequence of positive integers, got: {step}")
    if any(not isinstance(s, Integral) or s <= 0 for s in step):
        raise ValueError(f"`step` must be a positive integer or a sequence of positive integers, got: {step}")

    trailing = arr.shape[arr.ndim - m :] if m else ()
    if any(w > x for w, x in zip(window_shape[::-1], arr.shape[::-1])):
        raise ValueError(
            f"Each size of the window-shape must fit within the trailing dimensions of `arr`."
            f"{window_shape} does not fit in {trailing}"
        )

    if dilation is None:
        dilation = (1,) * m
    else:
        if isinstance(dilation, Integral):
            dilation = (int(dilation),) * m
        elif not hasattr(dilation, "__iter__"):
            raise TypeError(
                f"`dilation` must be None, a positive integer, or a sequence of positive integers, got: {dilation}"
            )
        if len(dilation) != m or any(not isinstance(d, Integral) or d <= 0 for d in dilation):
            raise ValueError(
                f"`dilation` must be None, a positive integer, or a sequence of positive integers "
                f"with the same length as `window_shape` ({window_shape}), got: {dilation}"
            )
        dilation = tuple(dilation)
        # the reference rejects w*d > dim (stricter than the true span (w-1)*d+1)
        if any(w * d > x for w, d, x in zip(window_shape[::-1], dilation[::-1], arr.shape[::-1])):
            raise ValueError(
                f"The dilated window ({tuple(w * d for w, d in zip(window_shape, dilation))}) must fit "
                f"within the trailing dimensions of `arr` ({trailing})"
            )

    if not arr.flags["C_CONTIGUOUS"]:
        arr = np.ascontiguousarray(arr)

    item = arr.itemsize
    elem_strides = _c_elem_strides(arr.shape)
    lead = arr.ndim - m
    grid, grid_strides, win_strides = [], [], []
    for k in range(m):
        x_k, es = arr.shape[lead + k], elem_strides[lead + k]
        span = (window_shape[k] - 1) * int(dilation[k]) + 1
        grid.append((x_k - span) // int(step[k]) + 1)
        grid_strides.append(int(step[k]) * es)
        win_strides.append(int(dilation[k]) * es)

    shape = tuple(grid) + arr.shape[:lead] + tuple(int(w) for w in window_shape)
    strides = tuple(item * s for s in (*grid_strides, *elem_strides[:lead], *win_strides))
    return as_strided(arr, shape=shape, strides=strides, writeable=False)


def _c_elem_strides(shape):
    """Row-major element strides as plain shape products (utils.py:207)."""
    out, acc = [], 1
    for n in reversed(shape):
        out.append(acc)
        acc *= int(n)
    return out[::-1]


# --------------------------------------------------------------------------- #
# convolution
# --------------------------------------------------------------------------- #
def _per_axis(value, m, name, lowest):
    """int-or-sequence -> int array of length m; AssertionError like
    src/mygrad/nnet/layers/conv.py:35-61."""
    if isinstance(value, Integral):
        arr = np.array((value,) * m)
    else:
        arr = np.array(value, dtype=int)
    if len(arr) != m or not all(v >= lowest and isinstance(v, Integral) for v in arr):
        raise AssertionError(f"bad {name}: {value}")
    return arr


def normalize_conv_args(m, stride, padding, dilation):
    dilation = _per_axis(dilation, m, "dilation", 1)
    padding = _per_axis(padding, m, "padding", 0)
    stride = _per_axis(stride, m, "stride", 1)
    return stride, padding, dilation


def conv_out_shape(x_spatial, w_spatial, stride, padding, dilation, validate=True):
    """Grid shape ``(G0, ...)``.  Exact-integer rule of conv.py:63-74 when
    ``validate``; otherwise the window helper's floor rule (utils.py:221-222)."""
    xs, ws = np.array(x_spatial), np.array(w_spatial)
    span = (ws - 1) * dilation + 1
    if validate:
        exact = (xs + 2 * padding - span) / stride + 1
        if not all(g.is_integer() and g > 0 for g in exact):
            raise ValueError(
                "Stride and kernel dimensions are incompatible: \n"
                f"Input dimensions: {tuple(xs)}\n"
                f"Stride dimensions: {tuple(stride)}\n"
                f"Kernel dimensions: {tuple(ws)}\n"
                f"Padding dimensions: {tuple(padding)}\n"
                f"Dilation dimensions: {tuple(dilation)}\n"
            )
    return tuple(int(g) for g in (xs + 2 * padding - span) // stride + 1)


def _zero_pad(x, padding):
    if not sum(padding):
        return x
    return np.pad(x, ((0, 0), (0, 0), *((int(p), int(p)) for p in padding)), mode="constant")


def conv_forward(x, w, *, stride, padding=0, dilation=1, validate=True):
    """``out[n,f,g] = sum_{c,t} w[f,c,t] * xpad[n,c,g*s+t*d]`` as pad -> window
    view -> tensordot -> move N to the front.  Follows conv.py:15-103."""
    assert x.ndim > 2 and x.ndim == w.ndim and x.shape[1] == w.shape[1]
    m = x.ndim - 2
    stride, padding, dilation = normalize_conv_args(m, stride, padding, dilation)
    conv_out_shape(x.shape[2:], w.shape[2:], stride, padding, dilation, validate)

    windows = window_view(_zero_pad(x, padding), w.shape[2:], tuple(stride), tuple(dilation))
    # w: (F, C, W...) ; windows: (G..., N, C, W...)  ->  (F, G..., N)
    w_axes = list(range(1, m + 2))
    win_axes = list(range(m + 1, 2 * m + 2))
    out = np.moveaxis(np.tensordot(w, windows, axes=[w_axes, win_axes]), -1, 0)
    return np.ascontiguousarray(out)


def conv_backward_x(grad, x_shape, x_dtype, w, *, stride, padding=0, dilation=1):
    """dx: GEMM ``(N, G..., F) @ (F, C*W...)`` then a col2im loop over grid
    positions in row-major order, accumulating in ``x_dtype``; padding cropped.
    Follows conv.py:114-138."""
    m = grad.ndim - 2
    stride, padding, dilation = normalize_conv_args(m, stride, padding, dilation)
    padded = tuple(x_shape[:2]) + tuple(int(n + 2 * p) for n, p in zip(x_shape[2:], padding))
    dx = np.zeros(padded, dtype=x_dtype)

    spread = np.tensordot(grad, w, axes=[[1], [0]])  # (N, G..., C, W...)
    taps = w.shape[2:]
    for g in np.ndindex(*grad.shape[2:]):
        where = tuple(
            slice(gk * sk, gk * sk + tk * dk, dk) for gk, tk, sk, dk in zip(g, taps, stride, dilation)
        )
        dx[(Ellipsis, *where)] += spread[(slice(None), *g, Ellipsis)]

    if sum(padding):
        dx = dx[(Ellipsis, *(slice(int(p), -int(p) if p else None) for p in padding))]
    return dx


def conv_backward_w(grad, x, w_shape, *, stride, padding=0, dilation=1):
    """dw: pad -> window view -> tensordot over ``(G..., N)``.  Follows
    conv.py:140-155."""
    m = grad.ndim - 2
    stride, padding, dilation = normalize_conv_args(m, stride, padding, dilation)
    windows = window_view(_zero_pad(x, padding), tuple(w_shape[2:]), tuple(stride), tuple(dilation))
    grad_axes = list(range(2, m + 2)) + [0]
    win_axes = list(range(m + 1))
    return np.tensordot(grad, windows, axes=[grad_axes, win_axes])


# --------------------------------------------------------------------------- #
# max-pool
# --------------------------------------------------------------------------- #
def _pool_args(x, pool, stride):
    """AssertionErrors of src/mygrad/nnet/layers/pooling.py:52-68."""
    if not isinstance(pool, (tuple, list, np.ndarray)) or not all(
        p >= 0 and isinstance(p, Integral) for p in pool
    ):
        raise AssertionError(f"bad pool: {pool}")
    pool = np.asarray(pool, dtype=int)
    if not all(p > 0 for p in pool):
        raise AssertionError(f"bad pool: {pool}")
    if x.ndim < len(pool):
        raise AssertionError("The number of pooled dimensions cannot exceed the dimensionality of the data.")
    if isinstance(stride, Integral):
        stride = np.array([stride] * len(pool))
    else:
        stride = np.asarray(stride, dtype=int)
    if len(stride) != len(pool) or not all(s >= 1 and isinstance(s, Integral) for s in stride):
        raise AssertionError(f"bad stride: {stride}")
    return pool, stride


def pool_out_shape(x_pooled_dims, pool, stride, validate=True):
    """Exact-integer rule of pooling.py:79-86 when ``validate``, else floor."""
    xs = np.array(x_pooled_dims)
    if validate:
        exact = (xs - pool) / stride + 1
        if not all(g.is_integer() and g > 0 for g in exact):
            raise ValueError(
                "Stride and kernel dimensions are incompatible: \n"
                f"Input dimensions: {tuple(xs)}\n"
                f"Stride dimensions: {tuple(stride)}\n"
                f"Pooling dimensions: {tuple(pool)}\n"
            )
    return tuple(int(g) for g in (xs - pool) // stride + 1)


def pool_forward(x, pool, stride, validate=True):
    """Windowed max over the trailing ``len(pool)`` axes.  Follows
    pooling.py:49-98."""
    pool, stride = _pool_args(x, pool, stride)
    m = len(pool)
    lead = x.ndim - m
    pool_out_shape(x.shape[lead:], pool, stride, validate)
    peak = window_view(x, tuple(pool), tuple(stride)).max(axis=tuple(range(-m, 0)))  # (G..., lead...)
    order = tuple(range(m, m + lead)) + tuple(range(m))
    return np.ascontiguousarray(peak.transpose(order))


def pool_argmax(x, pool, stride):
    """Per window, the position of its maximum inside the flattened (row-major) window:
    the first of equal maxima, the first NaN if there is one (``argmax(-1)`` of
    pooling.py:109-111), laid out ``(lead..., G...)`` like the pooled output."""
    pool, stride = _pool_args(x, pool, stride)
    m = len(pool)
    windows = window_view(x, tuple(pool), tuple(stride))  # (G..., lead..., P...)
    winner = windows.reshape(*windows.shape[: windows.ndim - m], -1).argmax(-1)  # (G..., lead...)
    nd = winner.ndim
    return winner.transpose(tuple(range(m, nd)) + tuple(range(m)))  # (lead..., G...)


def pool_backward(x, grad, pool, stride):
    """Route ``grad`` to the first-occurrence argmax of every window with an
    unbuffered, C-ordered ``np.add.at`` into a float64 image.  Follows
    pooling.py:100-149 (argmax :111, index algebra :119-144, add.at :147-148).
    The result is float64 whatever ``x.dtype`` is, like the reference."""
    pool, stride = _pool_args(x, pool, stride)
    m = len(pool)
    lead_shape, pooled_shape = x.shape[: x.ndim - m], x.shape[x.ndim - m :]

    winner = pool_argmax(x, pool, stride)  # (lead..., G...)
    grid = winner.shape[winner.ndim - m :]

    unit = _c_elem_strides(pooled_shape)  # flat offset of one step along each pooled axis
    inside = sum(a * u for a, u in zip(np.unravel_index(winner, tuple(pool)), unit))
    corner = sum(g * int(s) * u for g, s, u in zip(np.indices(grid), stride, unit))

    flat_shape = (*lead_shape, int(np.prod(grid)))
    where = np.indices(flat_shape)
    where[-1] = (inside + corner).reshape(flat_shape)

    dx = np.zeros((*lead_shape, int(np.prod(pooled_shape))))
    np.add.at(dx, tuple(where), grad.reshape(flat_shape))
    return dx.reshape(x.shape)


# ------------------------------------------------------------------ element-wise / sum
def multiply(a, b):
    """``Multiply.__call__``: ``np.multiply(a, b)`` (mygrad/math/arithmetic/ops.py:45-46)."""
    return np.multiply(a, b)


def multiply_backward(grad, a, b, index):
    """``Multiply.backward_var``: ``grad * b`` for the first operand, ``grad * a`` for the
    second (mygrad/math/arithmetic/ops.py:48-53)."""
    return grad * b if index == 0 else grad * a


def relu_forward(x):
    """``ReLu.__call__``: ``x * asarray(x > 0, dtype=x.dtype)``
    (mygrad/nnet/activations/relu.py:11-14)."""
    return x * np.asarray(x > 0, dtype=x.dtype)


def relu_backward(x, grad):
    """``ReLu.backward_var``: ``grad * back`` with ``back`` the forward pass's 0/1 mask
    (mygrad/nnet/activations/relu.py:16-17)."""
    return grad * np.asarray(x > 0, dtype=x.dtype)


def sum_axes(x, axis=None, keepdims=False):
    """``Sum.__call__``: ``np.sum(x, axis=axis, keepdims=keepdims)``
    (mygrad/operation_base.py:400-452 with ``numpy_func = np.sum``,
    mygrad/math/sequential/ops.py:120-121)."""
    return np.sum(x, axis=axis, keepdims=keepdims)


def sum_axes_backward(x, grad, axis=None, keepdims=False):
    """``Sum.backward_var`` (mygrad/math/sequential/ops.py:123-133): ``np.full`` for a sum
    over everything; otherwise the summed axes are put back into ``grad`` as axes of length
    one (unless they were kept) and the result is broadcast to ``x.shape``."""
    if axis is None:
        return np.full(x.shape, grad, dtype=x.dtype)
    axes = axis if hasattr(axis, "__iter__") else (axis,)
    grad = np.asarray(grad)
    if not keepdims:
        index = [slice(None)] * x.ndim
        for i in axes:
            index[i] = np.newaxis
        grad = grad[tuple(index)]
    return np.broadcast_to(grad, x.shape).astype(x.dtype, copy=False)


def reduce_broadcast(grad, var_shape):
    """Sum ``grad`` back to the shape of an operand that was broadcast
    (mygrad/_utils/__init__.py:131-168): first over the leading axes the operand lacks, then,
    keeping them, over the axes where the shapes differ."""
    if grad.shape == tuple(var_shape):
        return grad
    if grad.ndim != len(var_shape):
        if grad.ndim < len(var_shape):
            raise ValueError("the gradient has fewer axes than the operand it belongs to")
        grad = grad.sum(axis=tuple(range(grad.ndim - len(var_shape))))
    keep = tuple(n for n, i in enumerate(grad.shape) if i != var_shape[n])
    if keep:
        grad = grad.sum(axis=keep, keepdims=True)
    return grad


def multiply_broadcast_backward(grad, a, b, index):
    """What reaches operand ``index`` of a broadcasting ``Multiply``: ``grad * other``
    (mygrad/math/arithmetic/ops.py:48-53) summed back to the operand's shape by
    ``Operation.backward`` (mygrad/operation_base.py:89-97, :213)."""
    var, other = (a, b) if index == 0 else (b, a)
    return reduce_broadcast(grad * other, var.shape)


def sum_all(x):
    """``Sum.__call__`` with ``axis=None``: ``np.sum(x)``
    (mygrad/math/sequential/ops.py:120-121)."""
    return np.sum(x)


def sum_all_backward(x, grad):
    """``Sum.backward_var`` with ``axis=None``: ``np.full(a.shape, grad, dtype=a.dtype)``
    (mygrad/math/sequential/ops.py:123-126)."""
    return np.full(x.shape, grad, dtype=x.dtype)


# ------------------------------------------------------------------ batch normalisation
def _channel_axes(x):
    axes = tuple(i for i in range(x.ndim) if i != 1)
    keep = tuple(1 if n != 1 else d for n, d in enumerate(x.shape))
    return axes, keep


def batchnorm_forward(x, gamma=None, beta=None, *, eps):
    """BatchNorm.__call__ (src/mygrad/nnet/layers/batchnorm.py:43-74): returns
    ``(y, mean, var)`` with ``mean`` / ``var`` the (C,) arrays the operation binds."""
    x = np.asarray(x)
    axes, keep = _channel_axes(x)
    mean = x.mean(axis=axes)  # :58
    var = x.var(axis=axes)  # :59
    y = x - mean.reshape(keep)  # :61
    std = np.sqrt(var + eps).reshape(keep)  # :62
    y /= std  # :63
    if gamma is not None:
        y = y * np.asarray(gamma).reshape(keep)  # :69
    if beta is not None:
        y = y + np.asarray(beta).reshape(keep)  # :73
    return y, mean, var


def batchnorm_backward(grad, x, gamma=None, *, eps):
    """BatchNorm.backward_var for indices 0, 1, 2 (batchnorm.py:76-106): returns
    ``(dx, dgamma, dbeta)``; ``dgamma`` is the x_norm-weighted sum also when the forward
    pass had no gamma (the reference then never asks for it)."""
    x = np.asarray(x)
    grad = np.asarray(grad)
    axes, keep = _channel_axes(x)
    std = np.sqrt(x.var(axis=axes) + eps).reshape(keep)
    x_norm = (x - x.mean(axis=axes).reshape(keep)) / std
    count = x.size / x.shape[1]  # :81
    everything = list(range(x.ndim))
    dot = np.einsum(grad, everything, x_norm, everything, [1])  # :88, :102

    dx = grad - np.mean(grad, axis=axes, keepdims=True)  # :85
    rterm = x_norm * np.reshape(dot, keep)  # :87-90
    rterm /= count  # :91
    dx -= rterm  # :92
    dx /= std  # :93
    if gamma is not None:
        dx *= np.asarray(gamma).reshape(keep)  # :98
    return dx, dot, grad.sum(axis=axes)  # :99, :102, :106


# ------------------------------------------------------------------ repeat
def repeat_forward(a, repeats, axis=None):
    """Repeat.__call__ (src/mygrad/tensor_manip/tiling/ops.py:16-22)."""
    return np.repeat(np.asarray(a), repeats=repeats, axis=axis)


def repeat_backward(grad, a, repeats, axis=None):
    """Repeat.backward_var (tiling/ops.py:24-72): equal repeats sum a windowed view of the
    gradient whose windows span the runs of copies (:36-56); unequal repeats add the
    gradient into place through repeated flat indices (:58-72)."""
    a = np.asarray(a)
    grad = np.asarray(grad)
    if isinstance(repeats, Integral) or len(repeats) == 1:
        if not isinstance(repeats, Integral):
            (repeats,) = repeats
        if not repeats:
            return np.zeros(a.shape, dtype=grad.dtype)  # :32-34
        if axis is None:
            grad = grad.ravel()  # :38
            window_shape = (repeats,)
        else:
            window_shape = [1] * max(1, a.ndim)  # :43
            window_shape[axis] = repeats
            window_shape = tuple(window_shape)
        view = window_view(grad, window_shape, window_shape)  # :51-53
        out = view.sum(axis=tuple(range(-len(window_shape), 0)))  # :54
        if axis is None:
            out.shape = a.shape
        return out
    out = np.zeros((a.size,), dtype=grad.dtype)  # :67
    indices = np.arange(a.size).reshape(a.shape)
    indices = np.repeat(indices, repeats=repeats, axis=axis)
    np.add.at(out, indices.ravel(), grad.ravel())  # :70
    return out.reshape(a.shape)


# ------------------------------------------------------------------ matmul
def matmul_forward(a, b):
    """MatMul.__call__: ``np.matmul`` (src/mygrad/math/misc/ops.py:91-93)."""
    return np.matmul(np.asarray(a), np.asarray(b))


def _sum_to(arr, shape):
    """Undo broadcasting: what the reference's BinaryUfunc.backward does to a gradient whose
    shape exceeds its variable's (src/mygrad/operation_base.py:262-330, reduce_broadcast)."""
    arr = np.asarray(arr)
    extra = arr.ndim - len(shape)
    if extra:
        arr = arr.sum(axis=tuple(range(extra)))
    keep = tuple(i for i, n in enumerate(shape) if n == 1 and arr.shape[i] != 1)
    if keep:
        arr = arr.sum(axis=keep, keepdims=True)
    return arr


def matmul_backward(grad, a, b, index):
    """MatMul.backward_var (ops.py:95-126), reduced to the operand's shape."""
    a, b, grad = np.asarray(a), np.asarray(b), np.asarray(grad)
    if a.ndim == 1 and b.ndim == 1:  # :101-105
        return grad * b if index == 0 else grad * a
    if index == 0:
        if b.ndim > 1:  # :108-111
            if a.ndim == 1:
                grad = np.expand_dims(grad, -2)
            out = np.matmul(grad, b.swapaxes(-1, -2))
        else:  # :112-113
            out = np.expand_dims(grad, -1) * b
        if a.ndim == 1 and out.ndim > 1:
            out = out.reshape(*out.shape[:-2], out.shape[-1])
        return _sum_to(out, a.shape)
    if a.ndim > 1:  # :117-122
        if b.ndim == 1:
            grad = np.expand_dims(grad, -1)
        out = np.matmul(a.swapaxes(-1, -2), grad)
        if b.ndim == 1:
            out = out.squeeze(-1)
    else:  # :123-124
        out = a[:, np.newaxis] * np.expand_dims(grad, -2)
    return _sum_to(out, b.shape)


# ------------------------------------------------------------------ einsum
def einsum_forward(in_lbls, out_lbls, *arrays):
    """``EinSum.__call__``: ``np.einsum("<in_lbls>-><out_lbls>", *arrays)``
    (mygrad/linalg/ops.py:82-110); ``in_lbls`` is the comma-separated string."""
    return np.einsum(f"{in_lbls}->{out_lbls}", *arrays)


def einsum_backward(grad, index, in_lbls, out_lbls, arrays, factor=1):
    """``EinSum.backward_var`` (mygrad/linalg/ops.py:124-262): the operand's gradient is the
    summation of ``grad`` (in the operand's place, labelled like the result) with the other
    operands onto the operand's labels.  Labels of the operand that occur nowhere else were
    summed away on their own, so ``grad`` is first given an axis for each of them, broadcast
    to its length.  An operand with a repeated label (a trace or a diagonal) only ever read
    its diagonal: the summation is made onto the labels taken once (each at its last
    position, :21-42) and written along that diagonal into zeros (the reference writes
    through a strided view, :220-262).  ``factor`` is the number of times the same (tensor,
    labels) pair occurs among the operands (one gradient for all of them, scaled)."""
    lbls = in_lbls.split(",")
    full_lbl = lbls.pop(index)
    var_lbl = "".join(lbl for n, lbl in enumerate(full_lbl) if lbl not in full_lbl[n + 1 :])
    full_shape = arrays[index].shape
    size = dict(zip(full_lbl, full_shape))
    var_shape = tuple(size[lbl] for lbl in var_lbl)
    rest = tuple(a for n, a in enumerate(arrays) if n != index)
    known = set("".join(lbls)) | set(out_lbls)
    grad = np.asarray(grad)
    grad_lbl = out_lbls
    if set(var_lbl) - known:
        slots = [slice(None)] * grad.ndim
        shape = list(grad.shape)
        for n, lbl in enumerate(var_lbl):
            if lbl not in known:
                grad_lbl = grad_lbl[:n] + lbl + grad_lbl[n:]
                slots.insert(n, np.newaxis)
                shape.insert(n, var_shape[n])
        grad = np.broadcast_to(grad[tuple(slots)] if grad.ndim else grad, shape)
    back = np.einsum(",".join([grad_lbl] + lbls) + "->" + var_lbl, grad, *rest)
    back = reduce_broadcast(back, var_shape)
    if back.shape != var_shape:
        back = np.broadcast_to(back, var_shape)
    if var_lbl != full_lbl:
        along = np.indices(var_shape)
        placed = np.zeros(full_shape, dtype=back.dtype)
        placed[tuple(along[var_lbl.index(lbl)] for lbl in full_lbl)] = back
        back = placed
    return back * factor if factor > 1 else back
