"""Pins the CPU oracle: reference known answers, definition-level brute force,
adjoint identity, finite differences, and NumPy library routines on tiny cases.
A dropped term, a wrong sign/index or a transposed axis list fails one of these."""

import itertools
import math

import numpy as np
import pytest
from hypothesis import given, settings
from hypothesis import strategies as st

from oracle import brute, direct
from oracle import np_oracle as ora


# ----------------------------------------------------------------------------- window helper
def test_window_docstring_vectors(kats):
    case = kats["window"][0]
    x = np.arange(36).reshape(6, 6)
    y = ora.window_view(x, case["window_shape"], case["step"])
    assert list(y.shape) == case["shape"]
    for key, want in case["picks"].items():
        i, j = map(int, key.split(","))
        assert np.array_equal(y[i, j], np.array(want))


@pytest.mark.parametrize("dtype", [np.int8, np.int64, np.float16, np.float32, np.float64])
def test_window_memory_details(kats, dtype):
    case = kats["window"][1]
    want = np.array(case["view"])
    x = np.asfortranarray(np.arange(20).reshape(2, 10).astype(dtype))
    y = ora.window_view(x, (5,), 5)
    assert not y.flags["WRITEABLE"]
    assert np.array_equal(y, want)
    x = np.ascontiguousarray(np.arange(20).reshape(2, 10))
    y = ora.window_view(x, (5,), 5)
    assert not y.flags["WRITEABLE"] and np.shares_memory(x, y)
    assert np.array_equal(y, want)


@settings(deadline=None, max_examples=150)
@given(data=st.data(), shape=st.lists(st.integers(1, 7), min_size=1, max_size=4))
def test_window_matches_slicing(data, shape):
    x = np.arange(int(np.prod(shape))).reshape(shape)
    m = data.draw(st.integers(1, len(shape)))
    tail = shape[-m:]
    win = tuple(data.draw(st.integers(1, s)) for s in tail)
    step = tuple(data.draw(st.integers(1, s)) for s in tail)
    dil = tuple(data.draw(st.integers(1, s // w)) for s, w in zip(tail, win))
    y = ora.window_view(x, win, step, dil)
    grid = tuple((s - ((w - 1) * d + 1)) // st_ + 1 for s, w, st_, d in zip(tail, win, step, dil))
    assert y.shape == grid + tuple(shape[:-m]) + win
    for g in np.ndindex(*grid):
        sl = tuple(slice(i * s, i * s + w * d, d) for i, w, s, d in zip(g, win, step, dil))
        assert np.array_equal(y[g], x[(Ellipsis, *sl)])


@pytest.mark.parametrize(
    "kwargs",
    [
        dict(step=None),
        dict(step=-1),
        dict(window_shape=None),
        dict(window_shape=1),
        dict(window_shape=(1, 1, 1)),
        dict(window_shape=(-1, 1)),
        dict(window_shape=(1.0, 2.0)),
        dict(window_shape=(7, 5)),
        dict(dilation=-1),
        dict(dilation=(1, 0)),
        dict(dilation="aa"),
        dict(dilation=(1, 1, 1)),
        dict(dilation=1.0),
        dict(dilation=7),
        dict(dilation=(1, 7)),
    ],
)
def test_window_validation(kwargs):
    args = dict(arr=np.arange(36).reshape(6, 6), window_shape=(1, 1), step=1, dilation=None)
    args.update(kwargs)
    with pytest.raises((ValueError, TypeError)):
        ora.window_view(**args)


# ----------------------------------------------------------------------------- convolution
def test_conv_reference_known_answers(kats):
    for case in kats["conv"]:
        x, w = np.array(case["x"], dtype=float), np.array(case["w"], dtype=float)
        conf = dict(stride=tuple(case["stride"]), padding=tuple(case["padding"]), dilation=tuple(case["dilation"]))
        out = ora.conv_forward(x, w, **conf)
        assert np.array_equal(out, np.array(case["out"], dtype=float)), case["source"]
        if "dx_of_ones" in case:
            g = np.ones_like(out)
            dx = ora.conv_backward_x(g, x.shape, x.dtype, w, **conf)
            dw = ora.conv_backward_w(g, x, w.shape, **conf)
            assert np.array_equal(dx, np.array(case["dx_of_ones"], dtype=float))
            assert np.array_equal(dw, np.array(case["dw_of_ones"], dtype=float))


@pytest.mark.parametrize("m", [1, 2, 3, 4])
def test_conv_padding_only_image_is_zero(m):
    # reference tests/nnet/layers/test_conv.py:247-273: an empty image padded by p
    # and a kernel of extent 2p gives the single output 0.0
    rng = np.random.default_rng(m)
    pad = tuple(int(p) for p in rng.integers(1, 4, m))
    x = np.zeros((1, 1) + (0,) * m)
    w = rng.standard_normal((1, 1) + tuple(2 * p for p in pad))
    out = ora.conv_forward(x, w, stride=1, padding=pad)
    assert out.shape == (1,) * (m + 2) and out.item() == 0.0
    dx = ora.conv_backward_x(np.ones_like(out), x.shape, x.dtype, w, stride=1, padding=pad)
    assert dx.shape == x.shape


def _random_conv_case(rng, m):
    N, C, F = (int(v) for v in rng.integers(1, 4, 3))
    taps = tuple(int(v) for v in rng.integers(1, 4, m))
    dil = tuple(int(v) for v in rng.integers(1, 3, m))
    stride = tuple(int(v) for v in rng.integers(1, 4, m))
    pad = tuple(int(v) for v in rng.integers(0, 3, m))
    grid = tuple(int(v) for v in rng.integers(1, 4, m))
    X = tuple((g - 1) * s + (t - 1) * d + 1 - 2 * p for g, s, t, d, p in zip(grid, stride, taps, dil, pad))
    if any(v < 1 for v in X):
        return None
    # the reference's window helper rejects taps*dilation > padded extent (utils.py:188-196)
    if any(t * d > v + 2 * p for t, d, v, p in zip(taps, dil, X, pad)):
        return None
    x = rng.standard_normal((N, C, *X))
    w = rng.standard_normal((F, C, *taps))
    g = rng.standard_normal((N, F, *grid))
    return x, w, g, dict(stride=stride, padding=pad, dilation=dil)


@pytest.mark.parametrize("m", [1, 2, 3])
def test_conv_oracle_vs_bruteforce_and_direct(m):
    rng = np.random.default_rng(100 + m)
    done = 0
    while done < 12:
        case = _random_conv_case(rng, m)
        if case is None:
            continue
        x, w, g, conf = case
        s, p, d = conf["stride"], conf["padding"], conf["dilation"]
        out = ora.conv_forward(x, w, **conf)
        dx = ora.conv_backward_x(g, x.shape, x.dtype, w, **conf)
        dw = ora.conv_backward_w(g, x, w.shape, **conf)
        assert out.shape == g.shape
        np.testing.assert_allclose(out, brute.conv_forward(x, w, s, p, d), rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(dx, brute.conv_backward_x(g, x.shape, w, s, p, d), rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(dw, brute.conv_backward_w(g, x, w.shape, s, p, d), rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(out, direct.conv_forward(x, w, s, p, d), rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(dx, direct.conv_backward_x(g, x.shape, w, s, p, d), rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(dw, direct.conv_backward_w(g, x, w.shape, s, p, d), rtol=1e-12, atol=1e-12)
        done += 1


def test_conv_floor_placement_ignores_trailing_rows():
    # shapes the Operation-level validator rejects still run with the floor rule
    rng = np.random.default_rng(7)
    x = rng.standard_normal((2, 3, 8, 8))
    w = rng.standard_normal((4, 3, 3, 3))
    conf = dict(stride=2, padding=1, dilation=1)
    with pytest.raises(ValueError):
        ora.conv_forward(x, w, **conf)
    out = ora.conv_forward(x, w, validate=False, **conf)
    assert out.shape == (2, 4, 4, 4)
    np.testing.assert_allclose(out, brute.conv_forward(x, w, (2, 2), (1, 1), (1, 1)), rtol=1e-12, atol=1e-12)
    g = rng.standard_normal(out.shape)
    dx = ora.conv_backward_x(g, x.shape, x.dtype, w, **conf)
    np.testing.assert_allclose(dx, brute.conv_backward_x(g, x.shape, w, (2, 2), (1, 1), (1, 1)), rtol=1e-12, atol=1e-12)


def test_conv_adjoint_identity_and_finite_differences():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((3, 4, 9, 7))
    w = rng.standard_normal((5, 4, 3, 2))
    conf = dict(stride=(2, 1), padding=(1, 2), dilation=(1, 2))
    out = ora.conv_forward(x, w, **conf)
    g = rng.standard_normal(out.shape)
    dx = ora.conv_backward_x(g, x.shape, x.dtype, w, **conf)
    dw = ora.conv_backward_w(g, x, w.shape, **conf)
    lhs = np.vdot(out, g)
    assert abs(lhs - np.vdot(x, dx)) < 1e-10 * abs(lhs)
    assert abs(lhs - np.vdot(w, dw)) < 1e-10 * abs(lhs)
    # conv is linear in each argument: central differences are exact up to rounding
    h = 1e-3
    for _ in range(5):
        i = tuple(int(rng.integers(0, n)) for n in x.shape)
        e = np.zeros_like(x)
        e[i] = h
        num = (np.vdot(ora.conv_forward(x + e, w, **conf), g) - np.vdot(ora.conv_forward(x - e, w, **conf), g)) / (2 * h)
        assert abs(num - dx[i]) < 1e-8 * max(1.0, abs(dx[i]))
        j = tuple(int(rng.integers(0, n)) for n in w.shape)
        e = np.zeros_like(w)
        e[j] = h
        num = (np.vdot(ora.conv_forward(x, w + e, **conf), g) - np.vdot(ora.conv_forward(x, w - e, **conf), g)) / (2 * h)
        assert abs(num - dw[j]) < 1e-8 * max(1.0, abs(dw[j]))


def test_conv_dtype_rules():
    x = np.ones((1, 1, 5), dtype=np.float32)
    w = np.ones((1, 1, 2), dtype=np.float32)
    out = ora.conv_forward(x, w, stride=1)
    assert out.dtype == np.float32
    assert ora.conv_forward(x, w.astype(np.float64), stride=1).dtype == np.float64
    assert ora.conv_backward_x(out, x.shape, x.dtype, w, stride=1).dtype == np.float32


def test_conv_error_contract():
    x = np.zeros((1, 2, 2, 2))
    w = np.zeros((1, 2, 2, 2))
    with pytest.raises(ValueError):
        ora.conv_forward(x, np.zeros((1, 2, 3, 2)), stride=1, padding=0)
    with pytest.raises(AssertionError):
        ora.conv_forward(x, w, stride=0)
    with pytest.raises(AssertionError):
        ora.conv_forward(x, w, stride=[1, 2, 3])
    with pytest.raises(AssertionError):
        ora.conv_forward(x, w, stride=1, padding=-1)
    with pytest.raises(AssertionError):
        ora.conv_forward(x, w, stride=1, padding=[1, 2, 3])
    with pytest.raises(ValueError):
        ora.conv_forward(x, w, stride=3, padding=1)


# ----------------------------------------------------------------------------- max-pool
def test_pool_reference_known_answers(kats):
    for case in kats["pool"]:
        x = np.array(case["x"], dtype=case["dtype"])
        out = ora.pool_forward(x, tuple(case["pool"]), tuple(case["stride"]))
        assert out.dtype == x.dtype
        assert np.array_equal(out, np.array(case["out"], dtype=x.dtype)), case["source"]
        if case["grad"] is None:
            continue
        g = np.ones(out.shape) if case["grad"] == "ones" else np.arange(out.size).reshape(out.shape)
        dx = ora.pool_backward(x, g, tuple(case["pool"]), tuple(case["stride"]))
        assert dx.dtype == np.float64
        assert np.array_equal(dx, np.array(case["dx"], dtype=float)), case["source"]
        b_out, b_dx = brute.pool_forward_backward(x, g, case["pool"], case["stride"])
        assert np.array_equal(b_out, out) and np.array_equal(b_dx, dx)
        d_out, d_dx = direct.pool(x, g, case["pool"], case["stride"])
        assert np.array_equal(d_out, out) and np.array_equal(d_dx, dx)


@pytest.mark.parametrize("m,lead", [(1, (3,)), (2, (2, 2)), (3, (2,)), (2, ())])
def test_pool_ties_overlap_bit_exact_vs_bruteforce(m, lead):
    rng = np.random.default_rng(200 + m)
    for trial in range(10):
        pool = tuple(int(v) for v in rng.integers(1, 4, m))
        stride = tuple(int(v) for v in rng.integers(1, 4, m))
        grid = tuple(int(v) for v in rng.integers(1, 4, m))
        slack = tuple(int(v) for v in rng.integers(0, 2, m))  # rows the floor rule never covers
        X = tuple((g - 1) * s + p + e for g, s, p, e in zip(grid, stride, pool, slack))
        X = tuple(x if (x - p) // s + 1 == g else (g - 1) * s + p for x, p, s, g in zip(X, pool, stride, grid))
        dtype = np.float32 if trial % 2 else np.float64
        x = rng.integers(0, 4, (*lead, *X)).astype(dtype)  # few distinct values: ties everywhere
        g = rng.standard_normal((*lead, *grid)) * 10.0 ** rng.integers(-8, 8, (*lead, *grid))
        out = ora.pool_forward(x, pool, stride, validate=False)
        dx = ora.pool_backward(x, g, pool, stride)
        b_out, b_dx = brute.pool_forward_backward(x, g, pool, stride)
        assert np.array_equal(out.view(np.uint8), b_out.view(np.uint8))
        assert np.array_equal(dx.view(np.uint64), b_dx.view(np.uint64))
        d_out, d_dx = direct.pool(x, g.astype(dtype), pool, stride)
        dx_t = ora.pool_backward(x, g.astype(dtype), pool, stride)
        assert np.array_equal(d_out.view(np.uint8), out.view(np.uint8))
        assert np.array_equal(d_dx.view(np.uint64), dx_t.view(np.uint64))


def test_pool_argmax_is_the_first_of_equal_maxima_in_row_major_window_order():
    # the reference's docstring case (pooling.py:203-214): window [[2, 7], [5, 7]] holds 7 twice and
    # its gradient goes to row 1 of x, i.e. to offset 1 of the flattened window, not offset 3
    x = np.array([[0.0, 10.0, 8.0], [2.0, 7.0, 3.0], [5.0, 7.0, 20.0]])
    assert np.array_equal(ora.pool_argmax(x, (2, 2), 1), [[1, 0], [1, 3]])
    # the first NaN wins over everything, also over a later, larger value
    assert np.array_equal(ora.pool_argmax(np.array([1.0, np.nan, 5.0, np.nan, 2.0, 3.0]), (4,), 1), [1, 0, 1])
    # against loops: per window, walk it in row-major order and keep the first strict improvement
    rng = np.random.default_rng(207)
    for trial in range(8):
        m = 1 + trial % 3
        pool = tuple(int(v) for v in rng.integers(1, 4, m))
        stride = tuple(int(v) for v in rng.integers(1, 4, m))
        grid = tuple(int(v) for v in rng.integers(1, 4, m))
        X = tuple((g - 1) * s + p for g, s, p in zip(grid, stride, pool))
        x = rng.integers(0, 3, (2, *X)).astype(np.float64)
        got = ora.pool_argmax(x, pool, stride)
        assert got.shape == (2, *grid)
        for lead in range(2):
            for g in np.ndindex(*grid):
                best, where = None, -1
                for k, a in enumerate(np.ndindex(*pool)):
                    v = x[(lead, *(gi * si + ai for gi, si, ai in zip(g, stride, a)))]
                    if best is None or v > best:
                        best, where = v, k
                assert got[(lead, *g)] == where


def test_pool_accumulation_order_is_sequential_from_plus_zero():
    # one input element wins three overlapping windows; a sequential sum keeps
    # the 1.0 that a pairwise/reordered sum would lose
    x = np.array([0.0, 0.0, 9.0, 0.0, 0.0])
    g = np.array([1e16, 1.0, -1e16])
    dx = ora.pool_backward(x, g, (3,), (1,))
    assert dx[2] == (1e16 + 1.0) + -1e16 == 0.0
    g = np.array([1e16, -1e16, 1.0])
    assert ora.pool_backward(x, g, (3,), (1,))[2] == 1.0
    # an element whose only contribution is -0.0 ends as +0.0; untouched ones are +0.0
    dx = ora.pool_backward(np.array([1.0, 0.0]), np.array([-0.0]), (2,), (2,))
    assert not np.signbit(dx).any()


def test_pool_nan_routing():
    x = np.array([1.0, np.nan, 5.0, np.nan])
    assert np.isnan(ora.pool_forward(x, (4,), (1,))).all()
    dx = ora.pool_backward(x, np.array([2.0]), (4,), (1,))
    assert np.array_equal(dx, [0.0, 2.0, 0.0, 0.0])  # first NaN wins


def test_pool_error_contract():
    x = np.zeros((1, 2, 2, 2), dtype=np.float32)
    with pytest.raises(ValueError):
        ora.pool_forward(x, (3,) * 3, (1,) * 3)
    with pytest.raises(AssertionError):
        ora.pool_forward(x, (2,) * 3, (0,) * 3)
    with pytest.raises(AssertionError):
        ora.pool_forward(x, (2,) * 2, [1, 2, 3])
    with pytest.raises(ValueError):
        ora.pool_forward(x, (1,) * 3, (3,) * 3)


# ----------------------------------------------------------------- element-wise / sum
def test_relu_reference_docstring_vectors(kats):
    for case in kats["relu"]:
        for dtype in (np.float32, np.float64):
            x = np.array(case["x"], dtype=dtype)
            out = ora.relu_forward(x)
            assert np.array_equal(out, np.array(case["out"], dtype=dtype)), case["source"]
            assert np.array_equal(np.signbit(out), np.array(case["out_signbit"])), "negative inputs give -0.0"
            assert np.array_equal(ora.relu_backward(x, np.ones_like(x)), np.array(case["dx_of_ones"], dtype=dtype))


def test_relu_special_values_follow_the_multiplication():
    x = np.array([np.nan, np.inf, -np.inf, -0.0, 1e-45], dtype=np.float32)
    with np.errstate(invalid="ignore"):
        out = ora.relu_forward(x)
    assert np.isnan(out[0]) and out[1] == np.inf and np.isnan(out[2])  # -inf * 0 is NaN
    assert out[3] == 0.0 and np.signbit(out[3]) and out[4] == x[4]


def test_multiply_and_sum_oracle_closed_forms():
    import math

    rng = np.random.default_rng(7)
    a, b, g = (rng.standard_normal((3, 4, 5)) for _ in range(3))
    assert np.array_equal(ora.multiply(a, b), a * b)
    assert np.array_equal(ora.multiply_backward(g, a, b, 0), g * b)
    assert np.array_equal(ora.multiply_backward(g, a, b, 1), g * a)
    n = 100001
    assert ora.sum_all(np.arange(n, dtype=np.float64)) == n * (n - 1) / 2  # exact in float64
    x = rng.standard_normal(50000)
    assert abs(ora.sum_all(x) - math.fsum(x)) <= 1e-13 * np.sum(np.abs(x))
    assert np.array_equal(ora.sum_all_backward(a.astype(np.float32), np.float64(2.5)), np.full(a.shape, 2.5, np.float32))
    assert ora.sum_all_backward(a.astype(np.float32), 2.5).dtype == np.float32


# ----------------------------------------------------------------- batch normalisation
def test_batchnorm_reference_docstring_vector(kats):
    for case in kats["batchnorm"]:
        for dtype in (np.float32, np.float64):
            x = np.array(case["x"], dtype=dtype)
            y, mean, var = ora.batchnorm_forward(x, eps=case["eps"])
            assert y.dtype == dtype and mean.shape == var.shape == (x.shape[1],)
            assert np.allclose(y, np.array(case["out"]), rtol=0, atol=2 * 10.0 ** -case["decimals"] if dtype == np.float64 else 1e-6)


def _composed_batchnorm(x, gamma, beta, eps):
    """The second formulation the reference's tests compare against
    (tests/nnet/layers/test_batchnorm.py:13-48): variance as the mean of squared
    deviations, one division by the root."""
    axes = tuple(i for i in range(x.ndim) if i != 1)
    keep = tuple(1 if n != 1 else d for n, d in enumerate(x.shape))
    count = np.prod([x.shape[i] for i in axes])
    mean = x.sum(axis=axes, keepdims=True) / count
    var = ((x - mean) ** 2).sum(axis=axes, keepdims=True) / count
    out = (x - mean) / np.sqrt(var + eps)
    if gamma is not None:
        out = out * gamma.reshape(keep)
    if beta is not None:
        out = out + beta.reshape(keep)
    return out


BN_SHAPES = [(5, 3), (4, 3, 7), (3, 2, 5, 6), (2, 4, 3, 2, 3)]


@pytest.mark.parametrize("shape", BN_SHAPES)
@pytest.mark.parametrize("affine", [(False, False), (True, False), (False, True), (True, True)])
def test_batchnorm_forward_second_formulation_and_closed_forms(shape, affine):
    rng = np.random.default_rng([len(shape), int(np.prod(shape)), int(affine[0]), int(affine[1])])
    x = rng.uniform(-100, 100, shape)
    gamma = rng.uniform(-10, 10, shape[1]) if affine[0] else None
    beta = rng.uniform(-10, 10, shape[1]) if affine[1] else None
    eps = 1e-3
    y, mean, var = ora.batchnorm_forward(x, gamma, beta, eps=eps)
    assert np.allclose(y, _composed_batchnorm(x, gamma, beta, eps), rtol=1e-12, atol=1e-12)
    axes = tuple(i for i in range(x.ndim) if i != 1)
    g = np.ones(shape[1]) if gamma is None else gamma
    b = np.zeros(shape[1]) if beta is None else beta
    assert np.allclose(y.mean(axis=axes), b, atol=1e-12)
    assert np.allclose(y.var(axis=axes), g**2 * var / (var + eps), rtol=1e-11)
    assert np.allclose(mean, np.moveaxis(x, 1, 0).reshape(shape[1], -1).mean(axis=1))


@pytest.mark.parametrize("shape", BN_SHAPES)
@pytest.mark.parametrize("with_gamma", [False, True])
def test_batchnorm_backward_against_central_differences(shape, with_gamma):
    rng = np.random.default_rng([len(shape), int(np.prod(shape)), int(with_gamma), 77])
    x = rng.standard_normal(shape)
    gamma = rng.uniform(0.5, 2, shape[1]) * rng.choice([-1, 1], shape[1]) if with_gamma else None
    beta = rng.standard_normal(shape[1])
    grad = rng.standard_normal(shape)
    eps = 1e-2

    def loss(x_, gamma_, beta_):
        return float(np.sum(grad * ora.batchnorm_forward(x_, gamma_, beta_, eps=eps)[0]))

    dx, dgamma, dbeta = ora.batchnorm_backward(grad, x, gamma, eps=eps)
    h = 1e-6
    num_dx = np.zeros_like(x)
    for idx in np.ndindex(*shape):
        up, dn = x.copy(), x.copy()
        up[idx] += h
        dn[idx] -= h
        num_dx[idx] = (loss(up, gamma, beta) - loss(dn, gamma, beta)) / (2 * h)
    assert np.allclose(dx, num_dx, rtol=1e-6, atol=1e-7)

    base_gamma = np.ones(shape[1]) if gamma is None else gamma
    for c in range(shape[1]):
        e = np.zeros(shape[1])
        e[c] = h
        num_dgamma = (loss(x, base_gamma + e, beta) - loss(x, base_gamma - e, beta)) / (2 * h)
        num_dbeta = (loss(x, gamma, beta + e) - loss(x, gamma, beta - e)) / (2 * h)
        assert abs(dgamma[c] - num_dgamma) <= 1e-6 * max(1.0, abs(num_dgamma))
        assert abs(dbeta[c] - num_dbeta) <= 1e-6 * max(1.0, abs(num_dbeta))

    axes = tuple(i for i in range(x.ndim) if i != 1)
    assert np.allclose(dx.sum(axis=axes), 0, atol=1e-12)
    dx0, _, _ = ora.batchnorm_backward(grad, x, gamma, eps=0)
    xn0 = ora.batchnorm_forward(x, eps=0)[0]
    assert np.allclose((dx0 * xn0).sum(axis=axes), 0, atol=1e-11)


# ----------------------------------------------------------------- repeat
def test_repeat_reference_docstring_vectors(kats):
    for case in kats["repeat"]:
        out = ora.repeat_forward(np.array(case["a"]), case["repeats"], case["axis"])
        assert np.array_equal(out, np.array(case["out"])), case["source"]


def _repeat_backward_by_loops(grad, a_shape, repeats, axis):
    """dx[i] = sum of grad over the copies of entry i, located by repeating the flat indices."""
    size = int(np.prod(a_shape, dtype=np.int64))
    where = np.repeat(np.arange(size).reshape(a_shape), repeats, axis=axis).ravel()
    out = np.zeros(size, dtype=np.float64)
    for j, i in enumerate(where):
        out[i] += grad.ravel()[j]
    return out.reshape(a_shape)


REPEAT_CASES = [
    ((), 3, None),
    ((), 2, 0),
    ((5,), 0, None),
    ((5,), 4, 0),
    ((2, 3), 2, None),
    ((2, 3), 3, 1),
    ((2, 3, 4), 2, -2),
    ((2, 3, 4), [3], 0),
    ((2, 3), [1, 2], 0),
    ((2, 3), [0, 2, 5], 1),
    ((2, 2), [2, 0, 1, 3], None),
    ((3, 1, 2), [0, 0, 0], 0),
]


@pytest.mark.parametrize("shape, repeats, axis", REPEAT_CASES)
def test_repeat_backward_by_loops_and_adjoint(shape, repeats, axis):
    rng = np.random.default_rng([len(shape), int(np.prod(shape, dtype=np.int64)), 5])
    a = rng.standard_normal(shape)
    out = ora.repeat_forward(a, repeats, axis)
    grad = rng.standard_normal(out.shape)
    da = ora.repeat_backward(grad, a, repeats, axis)
    # a scalar repeated along axis 0 comes back as one entry; Operation.backward reshapes it
    assert da.shape == (a.shape or ((1,) if axis == 0 else ()))
    da = da.reshape(a.shape)
    assert np.allclose(da, _repeat_backward_by_loops(grad, a.shape, repeats, axis), rtol=0, atol=1e-13)
    assert abs(float(np.sum(out * grad)) - float(np.sum(a * da))) <= 1e-12 * max(1.0, float(np.sum(np.abs(out * grad))))


# ----------------------------------------------------------------- matmul
def test_matmul_reference_vectors(kats):
    for case in kats["matmul"]:
        if "a" in case:
            a, b = np.array(case["a"], dtype=float), np.array(case["b"], dtype=float)
            assert np.array_equal(ora.matmul_forward(a, b), np.array(case["out"], dtype=float)), case["source"]
            if "da" in case:
                g = np.ones_like(ora.matmul_forward(a, b))
                assert np.array_equal(ora.matmul_backward(g, a, b, 0), case["da"])
                assert np.array_equal(ora.matmul_backward(g, a, b, 1), case["db"])
        else:
            out = ora.matmul_forward(np.zeros(case["a_shape"]), np.zeros(case["b_shape"]))
            assert list(out.shape) == case["out_shape"]


MATMUL_SHAPES = [
    ((3, 4), (4, 5)),
    ((4,), (4, 5)),
    ((3, 4), (4,)),
    ((4,), (4,)),
    ((2, 3, 4), (4, 5)),
    ((3, 4), (2, 4, 5)),
    ((2, 3, 4), (2, 4, 5)),
    ((4,), (2, 3, 4, 5)),
    ((2, 3, 4), (4,)),
    ((2, 1, 3, 4), (2, 4, 5)),  # stacks that broadcast against each other
]


@pytest.mark.parametrize("sa, sb", MATMUL_SHAPES)
def test_matmul_backward_by_loops_and_adjoint(sa, sb):
    rng = np.random.default_rng([len(sa), len(sb), int(np.prod(sa)), int(np.prod(sb))])
    a, b = rng.standard_normal(sa), rng.standard_normal(sb)
    out = ora.matmul_forward(a, b)
    g = rng.standard_normal(out.shape)
    da, db = ora.matmul_backward(g, a, b, 0), ora.matmul_backward(g, a, b, 1)
    assert da.shape == a.shape and db.shape == b.shape
    inner = float(np.sum(out * g))
    assert abs(inner - float(np.sum(a * da))) <= 1e-12 * max(1.0, abs(inner))
    assert abs(inner - float(np.sum(b * db))) <= 1e-12 * max(1.0, abs(inner))
    # definition: out[..., i, k] = sum_j a[..., i, j] * b[..., j, k] on promoted operands
    a2 = a if a.ndim > 1 else a[None, :]
    b2 = b if b.ndim > 1 else b[:, None]
    want = np.einsum("...ij,...jk->...ik", a2, b2)
    if a.ndim == 1:
        want = want[..., 0, :]
    if b.ndim == 1:
        want = want[..., 0]
    assert np.allclose(out, want, rtol=1e-13, atol=1e-13)
    # d out[..., i, k] / d a[i, j] = b[j, k]: loops on the 2-D case
    if a.ndim == 2 and b.ndim == 2:
        loop_da = np.zeros_like(a)
        loop_db = np.zeros_like(b)
        for i in range(a.shape[0]):
            for j in range(a.shape[1]):
                for k in range(b.shape[1]):
                    loop_da[i, j] += g[i, k] * b[j, k]
                    loop_db[j, k] += a[i, j] * g[i, k]
        assert np.allclose(da, loop_da, atol=1e-13) and np.allclose(db, loop_db, atol=1e-13)


# ----------------------------------------------------------------- sums over axes, broadcasting
SUM_CASES = [((4, 5), 0, False), ((4, 5), -1, True), ((2, 3, 4), (0, 2), False), ((2, 3, 4), (1,), True),
             ((2, 1, 3, 2), (1, 3), False), ((3,), None, False), ((2, 3, 2, 2, 3), (1, 3), True), ((2, 3), (), False)]


@pytest.mark.parametrize("shape,axis,keepdims", SUM_CASES)
def test_sum_over_axes_against_exact_sums_and_loops(shape, axis, keepdims):
    rng = np.random.default_rng(len(shape) * 31 + (0 if axis is None else len(np.atleast_1d(axis))))
    x = rng.standard_normal(shape) * 10.0 ** rng.integers(-3, 4, shape)
    got = ora.sum_axes(x, axis, keepdims)
    axes = tuple(range(x.ndim)) if axis is None else tuple(a % x.ndim for a in np.atleast_1d(axis).astype(int))
    kept = [i for i in range(x.ndim) if i not in axes]
    want = np.zeros([shape[i] for i in kept])
    for k in np.ndindex(*want.shape):
        terms = []
        for r in np.ndindex(*[shape[i] for i in axes]):
            full = [0] * x.ndim
            for i, v in zip(kept, k):
                full[i] = v
            for i, v in zip(axes, r):
                full[i] = v
            terms.append(x[tuple(full)])
        want[k] = math.fsum(terms)
    assert got.shape == (tuple(1 if i in axes else n for i, n in enumerate(shape)) if keepdims else want.shape)
    assert np.allclose(got.reshape(want.shape), want, rtol=1e-13, atol=1e-13 * np.abs(x).sum())

    # gradient: every element of x receives the gradient of the entry it was added into
    g = rng.standard_normal(got.shape)
    back = ora.sum_axes_backward(x, g, axis, keepdims)
    assert back.shape == x.shape and back.dtype == x.dtype
    g_kept = g.reshape(want.shape)
    for full in np.ndindex(*shape):
        assert back[full] == g_kept[tuple(full[i] for i in kept)]
    # adjoint identity <sum(x), g> = <x, backward(g)>
    assert math.isclose(float(np.sum(got * g)), float(np.sum(x * back)), rel_tol=1e-10, abs_tol=1e-10)


def test_sum_axis_errors_are_numpys():
    x = np.zeros((2, 3))
    with pytest.raises(np.exceptions.AxisError):
        ora.sum_axes(x, 2)
    with pytest.raises(ValueError):
        ora.sum_axes(x, (0, 0))
    assert ora.sum_axes(np.array(3.0), 0) == 3.0  # NumPy lets a scalar be summed over axis 0


BROADCAST_CASES = [((4, 5), (5,)), ((4, 5), (4, 1)), ((2, 3, 4), (3, 1)), ((3, 1, 2), (1, 4, 1)), ((2, 3), ()),
                   ((1,), (2, 3)), ((2, 3, 4, 5), (1, 3, 1, 1)), ((5,), (5,))]


@pytest.mark.parametrize("sa,sb", BROADCAST_CASES)
def test_broadcast_multiply_gradients_against_loops_and_adjoints(sa, sb):
    rng = np.random.default_rng(len(sa) * 7 + len(sb))
    a, b = rng.standard_normal(sa), rng.standard_normal(sb)
    out = ora.multiply(a, b)
    shape = np.broadcast_shapes(sa, sb)
    assert out.shape == shape
    g = rng.standard_normal(shape)
    for index, (var, other) in enumerate(((a, b), (b, a))):
        got = ora.multiply_broadcast_backward(g, a, b, index)
        assert got.shape == var.shape
        # loops: walk every element of the result and add its term to the operand entry it read
        want = np.zeros(var.shape)
        pad_v = (1,) * (len(shape) - var.ndim) + var.shape
        pad_o = (1,) * (len(shape) - other.ndim) + other.shape
        v3, o3 = want.reshape(pad_v), other.reshape(pad_o)
        for full in np.ndindex(*shape):
            iv = tuple(0 if n == 1 else i for i, n in zip(full, pad_v))
            io = tuple(0 if n == 1 else i for i, n in zip(full, pad_o))
            v3[iv] += g[full] * o3[io]
        assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
        assert math.isclose(float(np.sum(out * g)), float(np.sum(var * got)), rel_tol=1e-9, abs_tol=1e-9)
    with pytest.raises(ValueError):
        ora.reduce_broadcast(np.zeros(3), (2, 3))


# ----------------------------------------------------------------- einsum
def _kat_operand(text):
    return np.asarray(eval(text, {"arange": lambda n: np.arange(float(n))}), dtype=np.float64)  # noqa: S307 (fixture text)


EINSUM_CASES = [
    ("ij,jk->ik", [(3, 4), (4, 5)]), ("ij,kj->ik", [(3, 4), (5, 4)]), ("bij,bjk->bik", [(2, 3, 4), (2, 4, 5)]),
    ("ijk,jil->kl", [(3, 4, 5), (4, 3, 2)]), ("i,i->", [(6,), (6,)]), ("i,j->ji", [(3,), (4,)]), ("ij->ji", [(3, 4)]),
    ("ijk->j", [(2, 3, 4)]), ("ij,jk->i", [(3, 4), (4, 5)]), ("ij,k->", [(2, 3), (4,)]), ("abc,cd->dab", [(2, 3, 4), (4, 5)]),
    (",ij->ij", [(), (2, 3)]), ("aib,ajb->abij", [(2, 3, 4), (2, 5, 4)]), ("ij->", [(3, 4)]), ("ij->ij", [(2, 3)]),
    ("ij,jk,kl->il", [(3, 4), (4, 5), (5, 2)]), ("bi,bj,bk->ijk", [(4, 2), (4, 3), (4, 5)]),
    # a label twice within an operand: traces and diagonals
    ("ii->", [(4, 4)]), ("ii->i", [(4, 4)]), ("iji->j", [(3, 2, 3)]), ("ijikik->jk", [(2, 3, 2, 4, 2, 4)]), ("ii,ij->j", [(3, 3), (3, 4)]),
    ("ijj,jk->ik", [(2, 3, 3), (3, 4)]), ("iij->", [(3, 3, 2)]),
]


def test_einsum_reference_docstring_vectors(kats):
    from numpy._core.einsumfunc import _parse_einsum_input

    for case in kats["einsum"]:
        arrays = [_kat_operand(t) for t in case["operands"]]
        in_lbls, out_lbls, _ = _parse_einsum_input([case["subscripts"], *arrays])
        got = ora.einsum_forward(in_lbls, out_lbls, *arrays)
        assert np.array_equal(got, np.array(case["out"], dtype=float)), case["source"]


@pytest.mark.parametrize("subscripts, shapes", EINSUM_CASES)
def test_einsum_backward_against_differences_adjoints_and_loops(subscripts, shapes):
    rng = np.random.default_rng(len(subscripts) * 13 + len(shapes))
    in_lbls, out_lbls = subscripts.split("->")
    arrays = [rng.standard_normal(s) for s in shapes]
    out = ora.einsum_forward(in_lbls, out_lbls, *arrays)
    g = rng.standard_normal(out.shape)
    lbls = in_lbls.split(",")
    sizes = {l: n for ls, a in zip(lbls, arrays) for l, n in zip(ls, a.shape)}
    every = sorted(sizes)
    for index, var in enumerate(arrays):
        back = ora.einsum_backward(g, index, in_lbls, out_lbls, arrays)
        assert back.shape == var.shape
        # adjoint identity (the summation is linear in each operand)
        assert math.isclose(float(np.sum(out * g)), float(np.sum(var * back)), rel_tol=1e-9, abs_tol=1e-9)
        # loops over the whole index space: each term of the result, times its gradient, goes to
        # the element of this operand that it read
        want = np.zeros(var.shape)
        for values in np.ndindex(*[sizes[l] for l in every]):
            at = dict(zip(every, values))
            term = g[tuple(at[l] for l in out_lbls)]
            for n, (ls, a) in enumerate(zip(lbls, arrays)):
                if n != index:
                    term = term * a[tuple(at[l] for l in ls)]
            want[tuple(at[l] for l in lbls[index])] += term
        assert np.allclose(back, want, rtol=1e-10, atol=1e-10)
        # central difference along one random direction
        direction = rng.standard_normal(var.shape)
        eps = 1e-6
        plus = [a + eps * direction if n == index else a for n, a in enumerate(arrays)]
        minus = [a - eps * direction if n == index else a for n, a in enumerate(arrays)]
        slope = float(np.sum((ora.einsum_forward(in_lbls, out_lbls, *plus) - ora.einsum_forward(in_lbls, out_lbls, *minus)) * g)) / (2 * eps)
        assert math.isclose(slope, float(np.sum(back * direction)), rel_tol=1e-6, abs_tol=1e-6)


@pytest.mark.parametrize("subscripts, shapes", [
    ("ij,ij->ij", [(2, 3), (1, 3)]), ("bij,bjk->bik", [(1, 3, 4), (5, 4, 2)]), ("ii,ij->j", [(1, 1), (3, 4)]),
    ("iji,ik->jk", [(1, 3, 1), (4, 2)]), ("ii,jj->ij", [(1, 1), (4, 4)]), ("iij,ik->jk", [(1, 1, 5), (6, 2)]),
])
def test_einsum_backward_of_broadcast_operands(subscripts, shapes):
    """An axis of length one under a label that is longer elsewhere: the gradient is summed over
    that label.  Pinned by the adjoint identity and central differences (np.einsum itself
    defines the forward values)."""
    rng = np.random.default_rng(len(subscripts) * 7 + len(shapes))
    in_lbls, out_lbls = subscripts.split("->")
    arrays = [rng.standard_normal(s) for s in shapes]
    out = ora.einsum_forward(in_lbls, out_lbls, *arrays)
    g = rng.standard_normal(out.shape)
    for index, var in enumerate(arrays):
        back = ora.einsum_backward(g, index, in_lbls, out_lbls, arrays)
        assert back.shape == var.shape
        assert math.isclose(float(np.sum(out * g)), float(np.sum(var * back)), rel_tol=1e-9, abs_tol=1e-9)
        for _ in range(3):
            direction = rng.standard_normal(var.shape)
            eps = 1e-6
            plus = [a + eps * direction if n == index else a for n, a in enumerate(arrays)]
            minus = [a - eps * direction if n == index else a for n, a in enumerate(arrays)]
            slope = float(np.sum((ora.einsum_forward(in_lbls, out_lbls, *plus) - ora.einsum_forward(in_lbls, out_lbls, *minus)) * g)) / (2 * eps)
            assert math.isclose(slope, float(np.sum(back * direction)), rel_tol=1e-6, abs_tol=1e-6)


def test_einsum_reference_docstring_trace_and_diagonal():
    a = np.arange(25.0).reshape(5, 5)
    assert ora.einsum_forward("ii", "", a) == 60.0  # linalg/funcs.py docstring: the trace
    assert np.array_equal(ora.einsum_forward("ii", "i", a), [0, 6, 12, 18, 24])  # and the diagonal
    # their gradients: ones on the diagonal, nothing off it
    assert np.array_equal(ora.einsum_backward(np.array(1.0), 0, "ii", "", [a]), np.eye(5))
    assert np.array_equal(ora.einsum_backward(np.arange(5.0), 0, "ii", "i", [a]), np.diag(np.arange(5.0)))


def test_einsum_backward_scales_a_repeated_pair():
    x = np.arange(4.0)
    assert np.array_equal(ora.einsum_backward(np.array(1.0), 0, "i,i", "", [x, x], factor=2), 2 * x)  # d(x.x)/dx
