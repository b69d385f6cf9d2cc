"""Definition-level loops for tiny inputs.  TEST INFRASTRUCTURE ONLY.

These share no code with ``np_oracle``: every output element is written from
the closed-form definition with explicit Python loops and scalar arithmetic, so
a transposed axis list or a wrong index in the NumPy restatement shows up as a
mismatch.  Sizes must stay tiny (pure Python).
"""

import itertools
import math

import numpy as np


def _grid(x_spatial, taps, stride, padding, dilation):
    return tuple(
        (x + 2 * p - ((t - 1) * d + 1)) // s + 1
        for x, t, s, p, d in zip(x_spatial, taps, stride, padding, dilation)
    )


def conv_forward(x, w, stride, padding, dilation):
    """out[n,f,g] = sum_{c,t} w[f,c,t] * x[n,c,g*s + t*d - p], zero outside x."""
    N, C = x.shape[:2]
    F = w.shape[0]
    X, T = x.shape[2:], w.shape[2:]
    G = _grid(X, T, stride, padding, dilation)
    out = np.zeros((N, F, *G), dtype=np.float64)
    for n, f in itertools.product(range(N), range(F)):
        for g in itertools.product(*map(range, G)):
            acc = 0.0
            for c in range(C):
                for t in itertools.product(*map(range, T)):
                    pos = tuple(gk * s + tk * d - p for gk, tk, s, d, p in zip(g, t, stride, dilation, padding))
                    if all(0 <= q < lim for q, lim in zip(pos, X)):
                        acc += float(w[(f, c, *t)]) * float(x[(n, c, *pos)])
            out[(n, f, *g)] = acc
    return out


def conv_backward_x(grad, x_shape, w, stride, padding, dilation):
    """dx[n,c,i] = sum over (f,t,g) with g*s + t*d - p == i of grad[n,f,g]*w[f,c,t]."""
    N, C = x_shape[:2]
    F = w.shape[0]
    X, T, G = tuple(x_shape[2:]), w.shape[2:], grad.shape[2:]
    dx = np.zeros(tuple(x_shape), dtype=np.float64)
    for n, c in itertools.product(range(N), range(C)):
        for i in itertools.product(*map(range, X)):
            acc = 0.0
            for f in range(F):
                for t in itertools.product(*map(range, T)):
                    g = []
                    for ik, tk, s, d, p, lim in zip(i, t, stride, dilation, padding, G):
                        num = ik + p - tk * d
                        if num % s or not 0 <= num // s < lim:
                            break
                        g.append(num // s)
                    else:
                        acc += float(grad[(n, f, *g)]) * float(w[(f, c, *t)])
            dx[(n, c, *i)] = acc
    return dx


def conv_backward_w(grad, x, w_shape, stride, padding, dilation):
    """dw[f,c,t] = sum_{n,g} grad[n,f,g] * x[n,c,g*s + t*d - p], zero outside x."""
    N, C = x.shape[:2]
    F = w_shape[0]
    X, T, G = x.shape[2:], tuple(w_shape[2:]), grad.shape[2:]
    dw = np.zeros(tuple(w_shape), dtype=np.float64)
    for f, c in itertools.product(range(F), range(C)):
        for t in itertools.product(*map(range, T)):
            acc = 0.0
            for n in range(N):
                for g in itertools.product(*map(range, G)):
                    pos = tuple(gk * s + tk * d - p for gk, tk, s, d, p in zip(g, t, stride, dilation, padding))
                    if all(0 <= q < lim for q, lim in zip(pos, X)):
                        acc += float(grad[(n, f, *g)]) * float(x[(n, c, *pos)])
            dw[(f, c, *t)] = acc
    return dw


def _first_max(values):
    """Index of the first element that no other element beats; the first NaN if
    there is one (what ``np.argmax`` documents)."""
    best = 0
    for k, v in enumerate(values):
        if math.isnan(v):
            return k
        if v > values[best]:
            best = k
    return best


def pool_forward_backward(x, grad, pool, stride):
    """(out, dx) of max-pool over the trailing ``len(pool)`` axes, windows placed
    with the floor rule.  Each window's gradient goes to the first (row-major
    inside the window) element that attains the maximum; ``dx`` starts from +0.0
    and takes the contributions window by window in row-major grid order, in
    float64."""
    m = len(pool)
    lead_shape, X = x.shape[: x.ndim - m], x.shape[x.ndim - m :]
    G = tuple((xk - pk) // sk + 1 for xk, pk, sk in zip(X, pool, stride))
    out = np.zeros((*lead_shape, *G), dtype=x.dtype)
    dx = np.zeros(x.shape, dtype=np.float64)
    for lead in itertools.product(*map(range, lead_shape)):
        for g in itertools.product(*map(range, G)):
            cells = [
                tuple(gk * sk + ak for gk, sk, ak in zip(g, stride, a))
                for a in itertools.product(*map(range, pool))
            ]
            vals = [float(x[(*lead, *cell)]) for cell in cells]
            k = _first_max(vals)
            out[(*lead, *g)] = x[(*lead, *cells[k])]
            if grad is not None:
                dx[(*lead, *cells[k])] = dx[(*lead, *cells[k])] + np.float64(grad[(*lead, *g)])
    return out, dx
