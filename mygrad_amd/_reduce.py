"""Sums over axes and broadcasts on device buffers, in terms of the two kernels that do
them: ``mg_sum_over`` (a C-contiguous array seen as ``(outer, n, inner)``, summed over the
middle axis or over the outer and inner ones) and ``mg_repeat_fwd`` (an axis of length one
repeated).  Neighbouring axes that are treated alike are merged first, so the usual
cases -- a bias gradient, a per-channel scale, a reduction over the last axes -- take one
launch; anything else takes one launch per remaining group of axes.

A product of two operands that broadcast against each other needs neither: ``multiply_plan``
gives the merged axes and the strides with which ``mg_multiply_broadcast`` reads each operand
where it lies.
"""

import ctypes

import numpy as np

from . import _device, _hip

__all__ = ["sum_axes", "broadcast", "permute", "multiply_plan", "multiply_broadcast"]


def _merge(pairs):
    """``[(size, kind), ...]`` without the axes of length one and with neighbours of one kind
    multiplied together."""
    merged = []
    for size, kind in pairs:
        if size == 1:
            continue
        if merged and merged[-1][1] == kind:
            merged[-1][0] *= size
        else:
            merged.append([int(size), kind])
    return merged


def _product(groups):
    total = 1
    for size, _ in groups:
        total *= size
    return total


def sum_axes(buf, shape, axes, dtype, times=None):
    """Device buffer with ``x.sum(axis=axes)`` of the C-contiguous ``x`` of ``shape`` in
    ``buf`` (``axes``: normalised, unique).  The array must not be empty.  With ``times``, the
    buffer of a ``y`` of the same shape, the sums are those of ``x * y`` (the product rounded
    before it is added, as if it had been formed first), in the same number of passes."""
    lib, code = _hip.lib(), _hip.dtype_code(dtype)

    def sum_over(outer, n, inner, over_middle, out):
        nonlocal times
        if times is None:
            _hip.check(lib.mg_sum_over(code, outer, n, inner, over_middle, buf.ptr, out.ptr))
        else:  # the first pass takes the product; what is left to sum afterwards is plain
            _hip.check(lib.mg_sum_product_over(code, outer, n, inner, over_middle, buf.ptr, times.ptr, out.ptr))
            times = None

    summed = set(axes)
    groups = _merge([(size, axis in summed) for axis, size in enumerate(shape)])
    if times is not None and not any(kind for _, kind in groups):
        raise ValueError("sum_axes with a second operand needs an axis to sum over")
    while any(kind for _, kind in groups):
        kinds = [kind for _, kind in groups]
        if kinds in ([True], [True, False], [False, True], [True, False, True]):
            # one kept group at most, summed groups around it: a single pass
            if kinds == [True] and times is None:  # everything that is left is summed: the whole-array kernel
                out = _device.DeviceBuffer(16)
                _hip.check(lib.mg_sum_all(code, groups[0][0], buf.ptr, out.ptr))
                return out
            elif kinds == [True]:  # of a product: one kept entry between nothing and the whole array
                outer, n, inner = 1, 1, groups[0][0]
            elif kinds == [True, False]:
                outer, n, inner = groups[0][0], groups[1][0], 1
            elif kinds == [False, True]:
                outer, n, inner = 1, groups[0][0], groups[1][0]
            else:
                outer, n, inner = (g[0] for g in groups)
            out = _device.DeviceBuffer(max(n * dtype.itemsize, 16))
            sum_over(outer, n, inner, 0, out)
            return out
        # several kept groups: take out the largest summed group, the rest next time round
        j = max((i for i, (_, kind) in enumerate(groups) if kind), key=lambda i: groups[i][0])
        outer, n, inner = _product(groups[:j]), groups[j][0], _product(groups[j + 1 :])
        out = _device.DeviceBuffer(max(outer * inner * dtype.itemsize, 16))
        sum_over(outer, n, inner, 1, out)
        buf = out
        groups = _merge([tuple(g) for g in groups[:j] + groups[j + 1 :]])
    return buf


def broadcast(buf, shape, to_shape, dtype):
    """Device buffer with ``np.broadcast_to(x, to_shape)`` made contiguous, for the
    C-contiguous ``x`` of ``shape`` in ``buf``.  ``to_shape`` must not be empty of elements."""
    shape = (1,) * (len(to_shape) - len(shape)) + tuple(shape)
    groups = _merge([(to, "copy" if have == to else "grow") for have, to in zip(shape, to_shape)])
    lib = _hip.lib()
    current = [size if kind == "copy" else 1 for size, kind in groups]
    for j, (size, kind) in enumerate(groups):
        if kind != "grow":
            continue
        outer = int(np.prod(current[:j], dtype=np.int64))
        inner = int(np.prod(current[j + 1 :], dtype=np.int64))
        out = _device.DeviceBuffer(max(outer * size * inner * dtype.itemsize, 16))
        _hip.check(lib.mg_repeat_fwd(dtype.itemsize, outer, 1, inner, size, size, None, buf.ptr, out.ptr))
        buf = out
        current[j] = size
    return buf


def permute(buf, shape, perm, dtype):
    """Device buffer with ``x.transpose(perm)`` made contiguous, for the C-contiguous ``x`` of
    ``shape`` in ``buf`` (not empty).  The same buffer comes back when nothing moves."""
    perm = tuple(int(p) for p in perm)
    moving = [p for p in perm if shape[p] != 1]
    if moving == sorted(moving):
        return buf
    nd = len(shape)
    out = _device.DeviceBuffer(max(int(np.prod(shape, dtype=np.int64)) * dtype.itemsize, 16))
    _hip.check(_hip.lib().mg_permute(dtype.itemsize, nd, (ctypes.c_int64 * nd)(*shape), (ctypes.c_int32 * nd)(*perm), buf.ptr, out.ptr))
    return out


def multiply_plan(a_shape, b_shape, shape):
    """``(extents, a_strides, b_strides)`` of ``a * b`` broadcast to ``shape``: neighbouring
    axes that both operands treat alike -- each is either there or broadcast -- are merged, axes
    of length one are dropped, strides are in elements of the C-contiguous operands and 0 where
    an operand is broadcast.  At least one axis comes back (``shape`` has no empty axis)."""
    nd = len(shape)
    a_shape = (1,) * (nd - len(a_shape)) + tuple(a_shape)
    b_shape = (1,) * (nd - len(b_shape)) + tuple(b_shape)
    groups = _merge([(size, (a_shape[i] == size, b_shape[i] == size)) for i, size in enumerate(shape)])
    if not groups:
        return [1], [0], [0]
    extents = [size for size, _ in groups]
    strides = ([], [])
    for which in (0, 1):
        step = 1
        for size, there in reversed(groups):
            strides[which].insert(0, step if there[which] else 0)
            if there[which]:
                step *= size
    return extents, strides[0], strides[1]


MAX_MULTIPLY_AXES = 6  # of mg_multiply_broadcast, after merging


def multiply_broadcast(a_buf, a_shape, b_buf, b_shape, shape, dtype):
    """Device buffer with ``a * b`` of ``shape``, for C-contiguous operands that broadcast to
    it, in one pass; ``None`` when the pattern has more axes than the kernel takes or the
    result 2^31 elements or more (the caller then spreads the operands first)."""
    extents, a_strides, b_strides = multiply_plan(a_shape, b_shape, shape)
    size = int(np.prod(shape, dtype=np.int64))
    if len(extents) > MAX_MULTIPLY_AXES or size >= 2**31:
        return None
    nd = len(extents)
    out = _device.DeviceBuffer(max(size * dtype.itemsize, 16))
    as_array = ctypes.c_int64 * nd
    _hip.check(
        _hip.lib().mg_multiply_broadcast(
            _hip.dtype_code(dtype), nd, as_array(*extents), as_array(*a_strides), as_array(*b_strides), a_buf.ptr, b_buf.ptr, out.ptr
        )
    )
    return out
