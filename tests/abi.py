"""Test helper: call the C-ABI kernels of libmygrad_hip.so on NumPy arrays
(upload -> kernel -> download), with the output grid chosen by the floor rule so
that shapes the Operation layer rejects can be exercised too."""

import numpy as np

from mygrad_amd import _device, _hip


def _grid(x_spatial, taps, stride, padding, dilation):
    return tuple(
        (int(x) + 2 * int(p) - ((int(t) - 1) * int(d) + 1)) // int(s) + 1
        for x, t, s, p, d in zip(x_spatial, taps, stride, padding, dilation)
    )


def _tup(v, m):
    return (int(v),) * m if np.isscalar(v) else tuple(int(i) for i in v)


def _up(arr):
    arr = np.ascontiguousarray(arr)
    buf = _device.DeviceBuffer(arr.nbytes)
    buf.upload(arr)
    return buf


def _down(buf, shape, dtype):
    out = np.empty(shape, dtype=dtype)
    buf.download_into(out)
    return out


def conv_desc(x_shape, w_shape, dtype, stride, padding, dilation):
    m = len(x_shape) - 2
    stride, padding, dilation = _tup(stride, m), _tup(padding, m), _tup(dilation, m)
    grid = _grid(x_shape[2:], w_shape[2:], stride, padding, dilation)
    return _hip.conv_desc(dtype, x_shape, w_shape, grid, stride, padding, dilation), grid


def conv_fwd(x, w, stride, padding=0, dilation=1):
    desc, grid = conv_desc(x.shape, w.shape, x.dtype, stride, padding, dilation)
    xb, wb = _up(x), _up(w)
    shape = (x.shape[0], w.shape[0], *grid)
    ob = _device.DeviceBuffer(int(np.prod(shape)) * x.dtype.itemsize)
    _hip.check(_hip.lib().mg_conv_fwd(desc, xb.ptr, wb.ptr, ob.ptr))
    return _down(ob, shape, x.dtype)


def conv_dgrad(grad, x_shape, w, stride, padding=0, dilation=1):
    desc, grid = conv_desc(x_shape, w.shape, w.dtype, stride, padding, dilation)
    assert tuple(grad.shape[2:]) == grid, (grad.shape, grid)
    gb, wb = _up(grad), _up(w)
    db = _device.DeviceBuffer(int(np.prod(x_shape)) * w.dtype.itemsize)
    _hip.check(_hip.lib().mg_conv_dgrad(desc, gb.ptr, wb.ptr, db.ptr))
    return _down(db, tuple(x_shape), w.dtype)


def conv_wgrad(grad, x, w_shape, stride, padding=0, dilation=1):
    desc, grid = conv_desc(x.shape, w_shape, x.dtype, stride, padding, dilation)
    assert tuple(grad.shape[2:]) == grid, (grad.shape, grid)
    gb, xb = _up(grad), _up(x)
    db = _device.DeviceBuffer(int(np.prod(w_shape)) * x.dtype.itemsize)
    _hip.check(_hip.lib().mg_conv_wgrad(desc, gb.ptr, xb.ptr, db.ptr))
    return _down(db, tuple(w_shape), x.dtype)


def pool_desc(x_shape, dtype, pool, stride, dx_dtype=None):
    m = len(pool)
    stride = _tup(stride, m)
    lead_shape, pooled = x_shape[: len(x_shape) - m], x_shape[len(x_shape) - m :]
    grid = tuple((int(x) - int(p)) // int(s) + 1 for x, p, s in zip(pooled, pool, stride))
    lead = int(np.prod(lead_shape, dtype=np.int64))
    return _hip.pool_desc(dtype, lead, pooled, pool, stride, grid, dx_dtype=dx_dtype), (*lead_shape, *grid)


def pool_fwd(x, pool, stride):
    desc, out_shape = pool_desc(x.shape, x.dtype, pool, stride)
    xb = _up(x)
    ob = _device.DeviceBuffer(int(np.prod(out_shape)) * x.dtype.itemsize)
    _hip.check(_hip.lib().mg_maxpool_fwd(desc, xb.ptr, ob.ptr))
    return _down(ob, out_shape, x.dtype)


def pool_bwd(x, grad, pool, stride, dx_dtype=None):
    dx_dtype = np.dtype(x.dtype if dx_dtype is None else dx_dtype)
    desc, out_shape = pool_desc(x.shape, x.dtype, pool, stride, dx_dtype=dx_dtype)
    assert tuple(grad.shape) == tuple(out_shape)
    xb, gb = _up(x), _up(np.ascontiguousarray(grad, dtype=x.dtype))
    db = _device.DeviceBuffer(x.size * dx_dtype.itemsize)
    _hip.check(_hip.lib().mg_maxpool_bwd(desc, xb.ptr, gb.ptr, db.ptr))
    return _down(db, x.shape, dx_dtype)


def pool_fwd_argmax(x, pool, stride):
    """(out, argmax): argmax holds one byte per window, its maximum's offset inside the window."""
    desc, out_shape = pool_desc(x.shape, x.dtype, pool, stride)
    xb = _up(x)
    windows = int(np.prod(out_shape))
    ob = _device.DeviceBuffer(max(windows * x.dtype.itemsize, 16))
    ab = _device.DeviceBuffer(max(windows, 16))
    _hip.check(_hip.lib().mg_maxpool_fwd_argmax(desc, xb.ptr, ob.ptr, ab.ptr))
    return _down(ob, out_shape, x.dtype), _down(ab, out_shape, np.uint8)


def pool_bwd_argmax(argmax, x_shape, x_dtype, grad, pool, stride, dx_dtype=None):
    x_dtype = np.dtype(x_dtype)
    dx_dtype = np.dtype(x_dtype if dx_dtype is None else dx_dtype)
    desc, out_shape = pool_desc(x_shape, x_dtype, pool, stride, dx_dtype=dx_dtype)
    assert tuple(grad.shape) == tuple(out_shape) == tuple(argmax.shape)
    ab, gb = _up(np.ascontiguousarray(argmax, dtype=np.uint8)), _up(np.ascontiguousarray(grad, dtype=x_dtype))
    db = _device.DeviceBuffer(int(np.prod(x_shape)) * dx_dtype.itemsize)
    _hip.check(_hip.lib().mg_maxpool_bwd_argmax(desc, ab.ptr, gb.ptr, db.ptr))
    return _down(db, tuple(x_shape), dx_dtype)


# ----------------------------------------------------------------- element-wise / sum
def multiply(a, b):
    ab, bb = _up(a), _up(b)
    ob = _device.DeviceBuffer(max(a.nbytes, 16))
    _hip.check(_hip.lib().mg_multiply(_hip.dtype_code(a.dtype), a.size, ab.ptr, bb.ptr, ob.ptr))
    return _down(ob, a.shape, a.dtype)


def multiply_broadcast(a, b):
    """a * b with NumPy's broadcasting through mg_multiply_broadcast (the merged axes and the
    strides come from the host's plan)."""
    from mygrad_amd import _reduce

    shape = np.broadcast_shapes(a.shape, b.shape)
    dtype = np.dtype(np.result_type(a, b))
    ob = _reduce.multiply_broadcast(_up(a.astype(dtype)), a.shape, _up(b.astype(dtype)), b.shape, shape, dtype)
    return None if ob is None else _down(ob, shape, dtype)


def relu_fwd(x):
    xb = _up(x)
    ob = _device.DeviceBuffer(max(x.nbytes, 16))
    _hip.check(_hip.lib().mg_relu_fwd(_hip.dtype_code(x.dtype), x.size, xb.ptr, ob.ptr))
    return _down(ob, x.shape, x.dtype)


def relu_bwd(x, grad):
    xb, gb = _up(x), _up(grad)
    ob = _device.DeviceBuffer(max(x.nbytes, 16))
    _hip.check(_hip.lib().mg_relu_bwd(_hip.dtype_code(x.dtype), x.size, xb.ptr, gb.ptr, ob.ptr))
    return _down(ob, x.shape, x.dtype)


def relu_fwd_mask(x):
    """(out, mask): mask holds one bit per element of x, bit i % 8 of byte i // 8."""
    xb = _up(x)
    ob = _device.DeviceBuffer(max(x.nbytes, 16))
    nbytes = (x.size + 7) // 8
    mb = _device.DeviceBuffer(max(nbytes, 16))
    _hip.check(_hip.lib().mg_relu_fwd_mask(_hip.dtype_code(x.dtype), x.size, xb.ptr, ob.ptr, mb.ptr))
    return _down(ob, x.shape, x.dtype), _down(mb, (nbytes,), np.uint8)


def relu_bwd_mask(mask, grad):
    mb, gb = _up(mask), _up(grad)
    ob = _device.DeviceBuffer(max(grad.nbytes, 16))
    _hip.check(_hip.lib().mg_relu_bwd_mask(_hip.dtype_code(grad.dtype), grad.size, mb.ptr, gb.ptr, ob.ptr))
    return _down(ob, grad.shape, grad.dtype)


def permute(x, perm):
    import ctypes

    nd = x.ndim
    xb = _up(x)
    ob = _device.DeviceBuffer(max(x.nbytes, 16))
    shape, order = (ctypes.c_int64 * max(nd, 1))(*x.shape), (ctypes.c_int32 * max(nd, 1))(*perm)
    _hip.check(_hip.lib().mg_permute(x.dtype.itemsize, nd, shape, order, xb.ptr, ob.ptr))
    return _down(ob, tuple(x.shape[p] for p in perm), x.dtype)


def strided_copy(x, shape, strides, out_elems=None):
    """gather (out_elems None): dense array of `shape` read from x at the strided offsets;
    scatter: x (dense, of `shape`) written at those offsets into zeros of out_elems elements."""
    import ctypes

    nd = len(shape)
    cs, ct = (ctypes.c_int64 * nd)(*shape), (ctypes.c_int64 * nd)(*strides)
    xb = _up(x)
    if out_elems is None:
        ob = _device.DeviceBuffer(max(int(np.prod(shape)) * x.dtype.itemsize, 16))
        _hip.check(_hip.lib().mg_strided_copy(x.dtype.itemsize, nd, cs, ct, x.size, 0, xb.ptr, ob.ptr))
        return _down(ob, tuple(shape), x.dtype)
    ob = _device.DeviceBuffer(max(out_elems * x.dtype.itemsize, 16))
    _hip.check(_hip.lib().mg_memset_zero(ob.ptr, out_elems * x.dtype.itemsize))
    _hip.check(_hip.lib().mg_strided_copy(x.dtype.itemsize, nd, cs, ct, out_elems, 1, xb.ptr, ob.ptr))
    return _down(ob, (out_elems,), x.dtype)


def sum_over(x3, over_middle):
    """x3:(outer, n, inner) -> sums over the middle axis (outer, inner) or over the other two (n,)."""
    outer, n, inner = x3.shape
    xb = _up(x3)
    out_shape = (outer, inner) if over_middle else (n,)
    ob = _device.DeviceBuffer(max(int(np.prod(out_shape)) * x3.dtype.itemsize, 16))
    _hip.check(_hip.lib().mg_sum_over(_hip.dtype_code(x3.dtype), outer, n, inner, int(over_middle), xb.ptr, ob.ptr))
    return _down(ob, out_shape, x3.dtype)


def sum_product_over(x3, y3, over_middle):
    """The same sums of x3 * y3, in one pass."""
    outer, n, inner = x3.shape
    xb, yb = _up(x3), _up(y3)
    out_shape = (outer, inner) if over_middle else (n,)
    ob = _device.DeviceBuffer(max(int(np.prod(out_shape)) * x3.dtype.itemsize, 16))
    _hip.check(_hip.lib().mg_sum_product_over(_hip.dtype_code(x3.dtype), outer, n, inner, int(over_middle), xb.ptr, yb.ptr, ob.ptr))
    return _down(ob, out_shape, x3.dtype)


def sum_all(x):
    xb = _up(x)
    ob = _device.DeviceBuffer(16)
    _hip.check(_hip.lib().mg_sum_all(_hip.dtype_code(x.dtype), x.size, xb.ptr, ob.ptr))
    return _down(ob, (), x.dtype)


def sum_all_static(x):
    """mg_sum_all through the entry point that allocates nothing (its chunk sums live in a fixed
    array of the library's device image)."""
    xb = _up(x)
    ob = _device.DeviceBuffer(16)
    _hip.check(_hip.lib().mg_sum_all_static(_hip.dtype_code(x.dtype), x.size, xb.ptr, ob.ptr))
    return _down(ob, (), x.dtype)


def fill_from(value, shape, dtype):
    vb = _up(np.asarray(value, dtype=dtype).reshape(1))
    n = int(np.prod(shape))
    ob = _device.DeviceBuffer(max(n * np.dtype(dtype).itemsize, 16))
    _hip.check(_hip.lib().mg_fill_from(_hip.dtype_code(dtype), n, vb.ptr, ob.ptr))
    return _down(ob, shape, dtype)


# ----------------------------------------------------------------- batch normalisation
def batchnorm_fwd(x, gamma=None, beta=None, *, eps):
    """-> (y, mean, var) of mg_batchnorm_fwd."""
    desc = _hip.bn_desc(x.shape, x.dtype, gamma is not None, beta is not None, eps)
    channels = x.shape[1]
    xb = _up(x)
    gb = _up(gamma.astype(x.dtype)) if gamma is not None else None
    bb = _up(beta.astype(x.dtype)) if beta is not None else None
    yb = _device.DeviceBuffer(max(x.nbytes, 16))
    mb = _device.DeviceBuffer(max(channels * x.itemsize, 16))
    vb = _device.DeviceBuffer(max(channels * x.itemsize, 16))
    _hip.check(
        _hip.lib().mg_batchnorm_fwd(
            desc, xb.ptr, gb.ptr if gb is not None else None, bb.ptr if bb is not None else None, yb.ptr, mb.ptr, vb.ptr
        )
    )
    return _down(yb, x.shape, x.dtype), _down(mb, (channels,), x.dtype), _down(vb, (channels,), x.dtype)


def batchnorm_bwd(grad, x, mean, var, gamma=None, *, eps, want=("x", "gamma", "beta")):
    """-> (dx, dgamma, dbeta) of mg_batchnorm_bwd; entries not in `want` are None."""
    desc = _hip.bn_desc(x.shape, x.dtype, gamma is not None, False, eps)
    channels = x.shape[1]
    xb, gradb, mb, vb = _up(x), _up(grad.astype(x.dtype)), _up(mean), _up(var)
    gb = _up(gamma.astype(x.dtype)) if gamma is not None else None
    small = max(channels * x.itemsize, 16)
    dxb = _device.DeviceBuffer(max(x.nbytes, 16)) if "x" in want else None
    dgb = _device.DeviceBuffer(small) if "gamma" in want else None
    dbb = _device.DeviceBuffer(small) if "beta" in want else None
    _hip.check(
        _hip.lib().mg_batchnorm_bwd(
            desc,
            xb.ptr,
            gradb.ptr,
            gb.ptr if gb is not None else None,
            mb.ptr,
            vb.ptr,
            dxb.ptr if dxb is not None else None,
            dgb.ptr if dgb is not None else None,
            dbb.ptr if dbb is not None else None,
        )
    )
    return (
        _down(dxb, x.shape, x.dtype) if dxb is not None else None,
        _down(dgb, (channels,), x.dtype) if dgb is not None else None,
        _down(dbb, (channels,), x.dtype) if dbb is not None else None,
    )


# ----------------------------------------------------------------- repeat, window copy
def _around_axis(shape, axis):
    if axis is None:
        return 1, int(np.prod(shape, dtype=np.int64)), 1
    axis = axis % len(shape)
    return (
        int(np.prod(shape[:axis], dtype=np.int64)),
        int(shape[axis]),
        int(np.prod(shape[axis + 1 :], dtype=np.int64)),
    )


def repeat_fwd(a, repeats, axis=None):
    """np.repeat through mg_repeat_fwd (a: at least 1-D)."""
    outer, n, inner = _around_axis(a.shape, axis)
    src_of = np.repeat(np.arange(n, dtype=np.int32), repeats)
    total = src_of.size
    uniform = np.ndim(repeats) == 0
    out_shape = (total,) if axis is None else (*a.shape[: axis % a.ndim], total, *a.shape[axis % a.ndim + 1 :])
    ab = _up(a)
    sb = None if uniform else _up(src_of)
    ob = _device.DeviceBuffer(max(int(np.prod(out_shape, dtype=np.int64)) * a.itemsize, 16))
    _hip.check(
        _hip.lib().mg_repeat_fwd(
            a.itemsize, outer, n, inner, int(repeats) if uniform else 0, total, sb.ptr if sb is not None else None, ab.ptr, ob.ptr
        )
    )
    return _down(ob, out_shape, a.dtype)


def repeat_bwd(grad, a_shape, repeats, axis=None):
    outer, n, inner = _around_axis(a_shape, axis)
    uniform = np.ndim(repeats) == 0
    offsets = None if uniform else np.concatenate([[0], np.cumsum(repeats)]).astype(np.int64)
    total = n * int(repeats) if uniform else int(offsets[-1])
    gb = _up(grad)
    fb = None if uniform else _up(offsets)
    ob = _device.DeviceBuffer(max(int(np.prod(a_shape, dtype=np.int64)) * grad.itemsize, 16))
    _hip.check(
        _hip.lib().mg_repeat_bwd(
            _hip.dtype_code(grad.dtype), outer, n, inner, int(repeats) if uniform else 0, total,
            fb.ptr if fb is not None else None, gb.ptr, ob.ptr,
        )
    )
    return _down(ob, tuple(a_shape), grad.dtype)


def window_gather(x, window, step, dilation):
    m = len(window)
    lead_shape, tail = x.shape[: x.ndim - m], x.shape[x.ndim - m :]
    grid = tuple((tail[k] - ((window[k] - 1) * dilation[k] + 1)) // step[k] + 1 for k in range(m))
    out_shape = grid + lead_shape + tuple(window)
    desc = _hip.window_desc(x.itemsize, int(np.prod(lead_shape, dtype=np.int64)), tail, window, step, dilation, grid)
    xb = _up(x)
    ob = _device.DeviceBuffer(max(int(np.prod(out_shape, dtype=np.int64)) * x.itemsize, 16))
    _hip.check(_hip.lib().mg_window_gather(desc, xb.ptr, ob.ptr))
    return _down(ob, out_shape, x.dtype)


# ----------------------------------------------------------------- matrix product
def matmul(a, x):
    """a:(M, K) @ x:(batch, K, N) -> (batch, M, N) through mg_matmul."""
    batch, K, N = x.shape
    M = a.shape[0]
    ab, xb = _up(a), _up(x)
    ob = _device.DeviceBuffer(max(batch * M * N * a.itemsize, 16))
    _hip.check(_hip.lib().mg_matmul(_hip.dtype_code(a.dtype), batch, M, K, N, ab.ptr, xb.ptr, ob.ptr))
    return _down(ob, (batch, M, N), a.dtype)


def matmul_batched(a, b, trans_a=False, trans_b=False):
    """op(a[p]) @ op(b[p]) for stacks a:(batch, M, K) -- (batch, K, M) with trans_a -- and
    b:(batch, K, N) -- (batch, N, K) with trans_b -- through mg_matmul_batched."""
    batch = a.shape[0]
    K, M = a.shape[1:] if trans_a else a.shape[:0:-1]
    N = b.shape[1] if trans_b else b.shape[2]
    ab, bb = _up(a), _up(b)
    ob = _device.DeviceBuffer(max(batch * M * N * a.itemsize, 16))
    _hip.check(_hip.lib().mg_matmul_batched(_hip.dtype_code(a.dtype), batch, M, K, N, int(trans_a), int(trans_b), ab.ptr, bb.ptr, ob.ptr))
    return _down(ob, (batch, M, N), a.dtype)


def matmul_da(grad, x, M):
    batch, K, N = x.shape
    gb, xb = _up(grad), _up(x)
    ob = _device.DeviceBuffer(max(M * K * x.itemsize, 16))
    _hip.check(_hip.lib().mg_matmul_da(_hip.dtype_code(x.dtype), batch, M, K, N, gb.ptr, xb.ptr, ob.ptr))
    return _down(ob, (M, K), x.dtype)


def matmul_dx(grad, a):
    batch, M, N = grad.shape
    K = a.shape[1]
    gb, ab = _up(grad), _up(a)
    ob = _device.DeviceBuffer(max(batch * K * N * a.itemsize, 16))
    _hip.check(_hip.lib().mg_matmul_dx(_hip.dtype_code(a.dtype), batch, M, K, N, gb.ptr, ab.ptr, ob.ptr))
    return _down(ob, (batch, K, N), a.dtype)
