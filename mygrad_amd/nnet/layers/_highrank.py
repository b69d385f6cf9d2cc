"""Convolutions over more than three axes, on the kernels for at most three.

The reference's ``ConvND`` takes any number of convolved axes
(``mygrad/nnet/layers/conv.py:23-29``; its own tests draw up to four,
``tests/nnet/layers/test_conv.py:247-273``); the kernels of ``libmygrad_hip.so`` take
one to three.  A rank-m convolution is a sum over the taps ``t0`` of its leading
convolved axis of rank-(m-1) convolutions::

    out[n, f, g0, g'] = sum_t0  conv(x_pad[n, :, g0*s0 + t0*d0, ...], w[:, :, t0, ...])[g']

and for a fixed ``t0`` the ``G0`` slices ``x_pad[:, :, g0*s0 + t0*d0]`` are simply ``G0``
more batch items.  So, per tap of the leading axis: gather those slices into a
``(N*G0, C, X1, ...)`` batch (one strided copy), gather ``w[:, :, t0]``, run the
rank-(m-1) convolution (recursively, until three axes are left) and add the results
up on the device in tap order -- a fixed order, so results repeat exactly.  The two
gradients decompose the same way: the input gradient scatters every tap's rank-(m-1)
input gradient back onto the rows ``g0*s0 + t0*d0`` of the padded ``dx`` it came from,
the filter gradient of tap ``t0`` is the rank-(m-1) filter gradient of the folded
batch.  Everything stays on the device (``mg_strided_copy``, ``mg_permute``,
``mg_accumulate``, ``mg_memset_zero`` and the convolution entry points); the cost is
one pass over ``x`` per leading tap, which is what a fourth convolved axis costs the
reference's ``tensordot`` too.
"""

import ctypes

import numpy as np

from ... import _device, _hip

__all__ = ["conv_forward", "conv_dgrad", "conv_wgrad"]


def _prod(values):
    total = 1
    for v in values:
        total *= int(v)
    return total


def _new(count, item):
    return _device.DeviceBuffer(max(int(count) * item, 16))


def _zeros(count, item):
    buf = _new(count, item)
    _hip.check(_hip.lib().mg_memset_zero(buf.ptr, int(count) * item))
    return buf


def _strided(dense_shape, strides, side_ptr, side_extent, item, scatter, dense_buf=None):
    """``scatter`` False: a new dense buffer of ``dense_shape`` read from the array at
    ``side_ptr`` through ``strides`` (in elements).  True: ``dense_buf`` written there."""
    nd = len(dense_shape)
    shape = (ctypes.c_int64 * nd)(*(int(n) for n in dense_shape))
    steps = (ctypes.c_int64 * nd)(*(int(s) for s in strides))
    lib = _hip.lib()
    if scatter:
        _hip.check(lib.mg_strided_copy(item, nd, shape, steps, int(side_extent), 1, dense_buf.ptr, side_ptr))
        return None
    out = _new(_prod(dense_shape), item)
    _hip.check(lib.mg_strided_copy(item, nd, shape, steps, int(side_extent), 0, side_ptr, out.ptr))
    return out


def _permute(buf, shape, perm, item):
    nd = len(shape)
    out = _new(_prod(shape), item)
    _hip.check(_hip.lib().mg_permute(item, nd, (ctypes.c_int64 * nd)(*(int(n) for n in shape)),
                                     (ctypes.c_int32 * nd)(*perm), buf.ptr, out.ptr))
    return out


def _add_into(acc, inc, count, dtype):
    code = _hip.dtype_code(dtype)
    _hip.check(_hip.lib().mg_accumulate(code, code, int(count), acc.ptr, inc.ptr))


class _Fold:
    """The leading convolved axis of one convolution taken apart: shapes of the folded
    rank-(m-1) problem and the strided views that connect it with the rank-m tensors."""

    def __init__(self, dtype, x_shape, w_shape, grid, stride, padding, dilation):
        self.dtype, self.item = dtype, dtype.itemsize
        self.N, self.C = int(x_shape[0]), int(x_shape[1])
        self.F = int(w_shape[0])
        self.X0, self.W0, self.G0 = int(x_shape[2]), int(w_shape[2]), int(grid[0])
        self.s0, self.p0, self.d0 = int(stride[0]), int(padding[0]), int(dilation[0])
        self.x_rest, self.w_rest, self.g_rest = tuple(x_shape[3:]), tuple(w_shape[3:]), tuple(grid[1:])
        self.R, self.Wr, self.Gr = _prod(self.x_rest), _prod(self.w_rest), _prod(self.g_rest)
        self.X0p = self.X0 + 2 * self.p0
        self.inner = dict(stride=tuple(stride[1:]), padding=tuple(padding[1:]), dilation=tuple(dilation[1:]))
        self.folded_x = (self.N * self.G0, self.C, *self.x_rest)
        self.folded_w = (self.F, self.C, *self.w_rest)
        self.padded_count = self.N * self.C * self.X0p * self.R

    # x (N, C, X0, R) <-> its copy padded with p0 zero rows at both ends of axis 0
    def pad_x(self, xb):
        if self.p0 == 0:
            return xb
        xp = _zeros(self.padded_count, self.item)
        _strided((self.N, self.C, self.X0, self.R), (self.C * self.X0p * self.R, self.X0p * self.R, self.R, 1),
                 xp.ptr + self.p0 * self.R * self.item, self.padded_count - self.p0 * self.R, self.item, True, xb)
        return xp

    def crop_x(self, xp):
        if self.p0 == 0:
            return xp
        return _strided((self.N, self.C, self.X0, self.R), (self.C * self.X0p * self.R, self.X0p * self.R, self.R, 1),
                        xp.ptr + self.p0 * self.R * self.item, self.padded_count - self.p0 * self.R, self.item, False)

    # the rows g0*s0 + t0*d0 (g0 = 0 .. G0-1) of the padded array as a (N, G0, C, R) batch
    def _rows_view(self, xp, t0):
        offset = t0 * self.d0 * self.R
        strides = (self.C * self.X0p * self.R, self.s0 * self.R, self.X0p * self.R, 1)
        return (self.N, self.G0, self.C, self.R), strides, xp.ptr + offset * self.item, self.padded_count - offset

    def rows(self, xp, t0):
        shape, strides, ptr, extent = self._rows_view(xp, t0)
        return _strided(shape, strides, ptr, extent, self.item, False)

    def add_to_rows(self, xp, t0, inc):
        """xp[n, c, g0*s0 + t0*d0, :] += inc[n, g0, c, :] (rows of one tap are distinct)."""
        shape, strides, ptr, extent = self._rows_view(xp, t0)
        cur = _strided(shape, strides, ptr, extent, self.item, False)
        _add_into(cur, inc, _prod(shape), self.dtype)
        _strided(shape, strides, ptr, extent, self.item, True, cur)

    # w[:, :, t0] as a contiguous (F, C, Wr) bank, and the way back
    def _tap_view(self, wb, t0):
        offset = t0 * self.Wr
        count = self.F * self.C * self.W0 * self.Wr
        return (self.F, self.C, self.Wr), (self.C * self.W0 * self.Wr, self.W0 * self.Wr, 1), wb.ptr + offset * self.item, count - offset

    def tap(self, wb, t0):
        if self.W0 == 1:
            return wb
        shape, strides, ptr, extent = self._tap_view(wb, t0)
        return _strided(shape, strides, ptr, extent, self.item, False)

    def put_tap(self, dwb, t0, part):
        shape, strides, ptr, extent = self._tap_view(dwb, t0)
        _strided(shape, strides, ptr, extent, self.item, True, part)

    # grad / out (N, F, G0, Gr) <-> the folded batch (N, G0, F, Gr)
    def fold_grad(self, gb):
        return _permute(gb, (self.N, self.F, self.G0, self.Gr), (0, 2, 1, 3), self.item)

    def unfold_out(self, acc):
        return _permute(acc, (self.N, self.G0, self.F, self.Gr), (0, 2, 1, 3), self.item)


def _direct(entry, dtype, x_shape, w_shape, grid, conf, a, b, out_count):
    desc = _hip.conv_desc(dtype, x_shape, w_shape, grid, conf["stride"], conf["padding"], conf["dilation"])
    out = _new(out_count, dtype.itemsize)
    _hip.check(getattr(_hip.lib(), entry)(desc, a.ptr, b.ptr, out.ptr))
    return out


def conv_forward(xb, wb, dtype, x_shape, w_shape, grid, stride, padding, dilation):
    """Device buffer with out:(N, F, *grid) for x:(N, C, X...) and w:(F, C, W...), any number
    of convolved axes (buffers in, buffer out)."""
    m = len(x_shape) - 2
    conf = dict(stride=tuple(stride), padding=tuple(padding), dilation=tuple(dilation))
    if m <= _hip.MG_MAX_ND:
        return _direct("mg_conv_fwd", dtype, x_shape, w_shape, grid, conf, xb, wb, x_shape[0] * w_shape[0] * _prod(grid))
    f = _Fold(dtype, x_shape, w_shape, grid, stride, padding, dilation)
    xp = f.pad_x(xb)
    count = f.N * f.G0 * f.F * f.Gr
    acc = None
    for t0 in range(f.W0):
        part = conv_forward(f.rows(xp, t0), f.tap(wb, t0), dtype, f.folded_x, f.folded_w, f.g_rest, **f.inner)
        if acc is None:
            acc = part
        else:
            _add_into(acc, part, count, dtype)
    return f.unfold_out(acc)


def conv_dgrad(gb, wb, dtype, x_shape, w_shape, grid, stride, padding, dilation):
    """Device buffer with dx:(N, C, X...) for grad:(N, F, *grid)."""
    m = len(x_shape) - 2
    conf = dict(stride=tuple(stride), padding=tuple(padding), dilation=tuple(dilation))
    if m <= _hip.MG_MAX_ND:
        return _direct("mg_conv_dgrad", dtype, x_shape, w_shape, grid, conf, gb, wb, _prod(x_shape))
    f = _Fold(dtype, x_shape, w_shape, grid, stride, padding, dilation)
    gf = f.fold_grad(gb)
    dxp = _zeros(f.padded_count, f.item)
    for t0 in range(f.W0):
        part = conv_dgrad(gf, f.tap(wb, t0), dtype, f.folded_x, f.folded_w, f.g_rest, **f.inner)
        f.add_to_rows(dxp, t0, part)
    return f.crop_x(dxp)


def conv_wgrad(gb, xb, dtype, x_shape, w_shape, grid, stride, padding, dilation):
    """Device buffer with dw:(F, C, W...) for grad:(N, F, *grid) and x."""
    m = len(x_shape) - 2
    conf = dict(stride=tuple(stride), padding=tuple(padding), dilation=tuple(dilation))
    if m <= _hip.MG_MAX_ND:
        return _direct("mg_conv_wgrad", dtype, x_shape, w_shape, grid, conf, gb, xb, _prod(w_shape))
    f = _Fold(dtype, x_shape, w_shape, grid, stride, padding, dilation)
    gf = f.fold_grad(gb)
    xp = f.pad_x(xb)
    dw = _new(_prod(w_shape), f.item)
    for t0 in range(f.W0):
        part = conv_wgrad(gf, f.rows(xp, t0), dtype, f.folded_x, f.folded_w, f.g_rest, **f.inner)
        if f.W0 == 1:
            return part
        f.put_tap(dw, t0, part)
    return dw
