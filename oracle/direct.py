"""ctypes binding of ``direct_ref.c``.  TEST INFRASTRUCTURE ONLY.

Definition-level loops in C with OpenMP, accumulating in double; independent of
the NumPy restatement and fast enough for the full benchmark shapes.
"""

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libdirect_ref.so")
_lib = None

_I64x3 = ctypes.c_int64 * 3


class _ConvShape(ctypes.Structure):
    _fields_ = [("N", ctypes.c_int64), ("C", ctypes.c_int64), ("F", ctypes.c_int64)] + [
        (k, _I64x3) for k in ("X", "W", "G", "S", "P", "D")
    ]


class _PoolShape(ctypes.Structure):
    _fields_ = [("lead", ctypes.c_int64)] + [(k, _I64x3) for k in ("X", "P", "S", "G")]


def build(force=False):
    """Compile ``libdirect_ref.so`` next to its source."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
        os.path.join(_HERE, "direct_ref.c")
    ):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libdirect_ref.so"])
    return _SO


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _pad3(values, fill):
    values = [int(v) for v in values]
    return _I64x3(*([fill] * (3 - len(values)) + values))


def _suffix(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    raise TypeError(f"direct reference handles float32/float64 only, got {dtype}")


def _conv_shape(x_shape, w_shape, stride, padding, dilation):
    m = len(x_shape) - 2
    assert 1 <= m <= 3 and len(w_shape) == m + 2
    X, W = x_shape[2:], w_shape[2:]
    G = [(x + 2 * p - ((t - 1) * d + 1)) // s + 1 for x, t, s, p, d in zip(X, W, stride, padding, dilation)]
    sh = _ConvShape(
        N=x_shape[0], C=x_shape[1], F=w_shape[0],
        X=_pad3(X, 1), W=_pad3(W, 1), G=_pad3(G, 1),
        S=_pad3(stride, 1), P=_pad3(padding, 0), D=_pad3(dilation, 1),
    )
    return sh, tuple(G)


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data)


def conv_forward(x, w, stride, padding, dilation):
    x, w = np.ascontiguousarray(x), np.ascontiguousarray(w)
    sh, G = _conv_shape(x.shape, w.shape, stride, padding, dilation)
    out = np.empty((x.shape[0], w.shape[0], *G), dtype=np.float64)
    getattr(_load(), "direct_conv_fwd_" + _suffix(x.dtype))(ctypes.byref(sh), _ptr(x), _ptr(w), _ptr(out))
    return out


def conv_backward_x(grad, x_shape, w, stride, padding, dilation):
    grad, w = np.ascontiguousarray(grad), np.ascontiguousarray(w)
    sh, G = _conv_shape(tuple(x_shape), w.shape, stride, padding, dilation)
    assert tuple(grad.shape[2:]) == G, (grad.shape, G)
    dx = np.empty(tuple(x_shape), dtype=np.float64)
    getattr(_load(), "direct_conv_dx_" + _suffix(w.dtype))(ctypes.byref(sh), _ptr(grad), _ptr(w), _ptr(dx))
    return dx


def conv_backward_w(grad, x, w_shape, stride, padding, dilation):
    grad, x = np.ascontiguousarray(grad), np.ascontiguousarray(x)
    sh, G = _conv_shape(x.shape, tuple(w_shape), stride, padding, dilation)
    assert tuple(grad.shape[2:]) == G, (grad.shape, G)
    dw = np.empty(tuple(w_shape), dtype=np.float64)
    getattr(_load(), "direct_conv_dw_" + _suffix(x.dtype))(ctypes.byref(sh), _ptr(grad), _ptr(x), _ptr(dw))
    return dw


def pool(x, grad, pool, stride):
    """(out, dx) with dx in float64; ``grad=None`` gives (out, None)."""
    x = np.ascontiguousarray(x)
    m = len(pool)
    assert 1 <= m <= 3
    lead_shape, X = x.shape[: x.ndim - m], x.shape[x.ndim - m :]
    G = [(xk - pk) // sk + 1 for xk, pk, sk in zip(X, pool, stride)]
    sh = _PoolShape(
        lead=int(np.prod(lead_shape, dtype=np.int64)),
        X=_pad3(X, 1), P=_pad3(pool, 1), S=_pad3(stride, 1), G=_pad3(G, 1),
    )
    out = np.empty((*lead_shape, *G), dtype=x.dtype)
    dx = None
    gptr = dptr = ctypes.c_void_p(None)
    if grad is not None:
        grad = np.ascontiguousarray(grad, dtype=x.dtype)
        dx = np.empty(x.shape, dtype=np.float64)
        gptr, dptr = _ptr(grad), _ptr(dx)
    getattr(_load(), "direct_pool_" + _suffix(x.dtype))(ctypes.byref(sh), _ptr(x), gptr, _ptr(out), dptr)
    return out, dx
