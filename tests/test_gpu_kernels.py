"""Parity of the HIP kernels (called through the C ABI) against the CPU oracle.

Bars: pooling bit-exact (raw bit patterns); convolution
max|gpu - ref| / max|ref| <= 1e-10 in float64 and <= 2e-4 in float32.
"""

import os

import numpy as np
import pytest

from oracle import direct
from oracle import np_oracle as ora

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float64): 1e-10, np.dtype(np.float32): 2e-4}


@pytest.fixture(scope="module")
def abi():
    import mygrad_amd

    if not mygrad_amd.is_available():
        pytest.fail("libmygrad_hip.so / gfx950 device not available: the GPU tests need both")
    from tests import abi as module

    return module


def rel_err(got, want):
    scale = float(np.max(np.abs(want))) or 1.0
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) / scale


def bits(a):
    return a.view(np.uint32 if a.dtype == np.float32 else np.uint64)


# ----------------------------------------------------------------------------- pooling
class _Remembered:
    """The pair of entry points that keeps each window's argmax from the forward pass,
    behind the calling convention of the pair that recomputes it from x."""

    def __init__(self, abi):
        self.abi = abi

    def pool_fwd(self, x, pool, stride):
        out, argmax = self.abi.pool_fwd_argmax(x, pool, stride)
        # what was recorded is np.argmax over each flattened window (pooling.py:109-111)
        if x.size <= 1 << 22:
            assert argmax.dtype == np.uint8 and np.array_equal(argmax, ora.pool_argmax(x, pool, stride))
        return out

    def pool_bwd(self, x, grad, pool, stride, dx_dtype=None):
        _, argmax = self.abi.pool_fwd_argmax(x, pool, stride)
        return self.abi.pool_bwd_argmax(argmax, x.shape, x.dtype, grad, pool, stride, dx_dtype=dx_dtype)


@pytest.fixture(params=["recompute", "remember"])
def pools(request, abi):
    return abi if request.param == "recompute" else _Remembered(abi)


def test_pool_reference_known_answers(pools, kats):
    for case in kats["pool"]:
        x = np.array(case["x"], dtype=case["dtype"])
        pool, stride = tuple(case["pool"]), tuple(case["stride"])
        out = pools.pool_fwd(x, pool, stride)
        assert np.array_equal(out, np.array(case["out"], dtype=x.dtype)), case["source"]
        if case["grad"] is None:
            continue
        g = np.ones(out.shape) if case["grad"] == "ones" else np.arange(out.size).reshape(out.shape)
        for dx_dtype in (x.dtype, np.float64):
            dx = pools.pool_bwd(x, g, pool, stride, dx_dtype=dx_dtype)
            assert dx.dtype == dx_dtype
            assert np.array_equal(dx, np.array(case["dx"], dtype=float)), case["source"]


@pytest.mark.parametrize("m,lead", [(1, (3,)), (1, (2, 5)), (2, (2, 3)), (3, (2,)), (2, ()), (3, (1, 2))])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_pool_ties_and_overlap_bit_exact(pools, m, lead, dtype):
    rng = np.random.default_rng(300 + 10 * m + len(lead))
    for trial in range(12):
        pool = tuple(int(v) for v in rng.integers(1, 5, m))
        stride = tuple(int(v) for v in rng.integers(1, 5, m))
        grid = tuple(int(v) for v in rng.integers(1, 9, m))
        slack = tuple(int(v) for v in rng.integers(0, 2, m))
        X = tuple((g - 1) * s + p + (e if e < s else 0) for g, s, p, e in zip(grid, stride, pool, slack))
        print("pool case", m, lead, dtype.__name__, pool, stride, X, flush=True)
        if trial % 3 == 0:
            x = rng.standard_normal((*lead, *X)).astype(dtype)
        else:
            x = rng.integers(0, 4, (*lead, *X)).astype(dtype)  # few distinct values: ties everywhere
        out_shape = (*lead, *(((xk - pk) // sk + 1) for xk, pk, sk in zip(X, pool, stride)))
        g = (rng.standard_normal(out_shape) * 10.0 ** rng.integers(-6, 6, out_shape)).astype(dtype)
        want_out = ora.pool_forward(x, pool, stride, validate=False)
        want_dx = ora.pool_backward(x, g, pool, stride)  # float64
        out = pools.pool_fwd(x, pool, stride)
        assert np.array_equal(bits(out), bits(want_out))
        dx64 = pools.pool_bwd(x, g, pool, stride, dx_dtype=np.float64)
        assert np.array_equal(bits(dx64), bits(want_dx))
        dx = pools.pool_bwd(x, g, pool, stride)
        assert np.array_equal(bits(dx), bits(want_dx.astype(dtype)))
        hits = pools.pool_bwd(x, np.ones(out_shape, dtype), pool, stride)
        assert np.array_equal(hits, ora.pool_backward(x, np.ones(out_shape), pool, stride))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("lead,X,pool,stride", [
    ((3, 2), (11, 16), (3, 3), (2, 2)),   # an odd number of rows: the last row group is half empty
    ((5,), (56, 56), (3, 3), (2, 2)),     # the benchmark's plane (rows 55 and columns 55 are never covered)
    ((2,), (9, 12), (3, 3), (1, 1)),      # every element under up to nine windows
    ((4,), (7, 8), (2, 2), (1, 1)),
    ((2,), (3, 6, 8), (1, 3, 3), (1, 2, 2)),  # a leading pooled axis of extent one folds into the planes
    ((1,), (3, 4), (3, 3), (2, 2)),       # a single window per plane
    # exact window grids over an odd last extent (what the reference's validator admits for 3 x 3 windows
    # placed every other column): rows start on no 16-byte boundary and end in a short piece
    ((3, 2), (11, 15), (3, 3), (2, 2)),
    ((5,), (55, 55), (3, 3), (2, 2)),     # the valid neighbour of the benchmark's plane
    ((2,), (5, 7), (3, 3), (2, 2)),       # short pieces of three (float32) and one (float64) columns
    ((2,), (5, 5), (3, 3), (2, 2)),       # of one column in either precision
    ((3,), (9, 13), (3, 3), (1, 1)),
    ((3,), (7, 9), (2, 2), (1, 1)),
    ((2,), (5, 6), (3, 3), (1, 1)),       # a short piece of two float32 columns
    ((2,), (3, 3), (3, 3), (2, 2)),       # a float32 row shorter than one piece
    # 3 x 3 x 3 windows at every other position: the same kernels with a pooled leading axis
    ((2, 2), (7, 9, 13), (3, 3, 3), (2, 2, 2)),
    ((3,), (5, 7, 8), (3, 3, 3), (2, 2, 2)),     # flooring placement along the last axis
    ((2,), (8, 10, 12), (3, 3, 3), (2, 2, 2)),   # the last plane, row and column are never covered
    ((1,), (9, 65, 65), (3, 3, 3), (2, 2, 2)),   # planes too large for a band in LDS
    ((2,), (3, 5, 9), (3, 3, 3), (2, 2, 2)),     # a single window plane
])
def test_pool_backward_gather_for_windows_known_at_compile_time(pools, dtype, lead, X, pool, stride):
    """2-D windows of 3x3 / stride 2, 3x3 / stride 1 and 2x2 / stride 1 over rows of whole 16-byte
    pieces: the backward pass from the recorded argmax gathers per element in registers.  Ties,
    NaNs, gradients of -0.0 and huge / tiny magnitudes (the order of the additions shows), the
    float64 dx of a float32 input."""
    rng = np.random.default_rng(370 + X[-1] + X[-2])
    for trial in range(5):
        if trial == 0:
            x = rng.standard_normal((*lead, *X)).astype(dtype)
        else:
            x = rng.integers(0, 3, (*lead, *X)).astype(dtype)
        if trial == 2:
            x[rng.random(x.shape) < 0.1] = np.nan
        out_shape = (*lead, *(((xk - pk) // sk + 1) for xk, pk, sk in zip(X, pool, stride)))
        g = (rng.standard_normal(out_shape) * 10.0 ** rng.integers(-6, 6, out_shape)).astype(dtype)
        if trial == 3:
            g = rng.choice(np.array([1e16, 1.0, -1e16], dtype=dtype), out_shape)  # sums that depend on their order
        g[rng.random(out_shape) < 0.2] = -0.0
        want_dx = ora.pool_backward(x, g, pool, stride)  # float64
        assert np.array_equal(bits(pools.pool_fwd(x, pool, stride)), bits(ora.pool_forward(x, pool, stride, validate=False)))
        assert np.array_equal(bits(pools.pool_bwd(x, g, pool, stride, dx_dtype=np.float64)), bits(want_dx))
        assert np.array_equal(bits(pools.pool_bwd(x, g, pool, stride)), bits(want_dx.astype(dtype)))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("lead,X,pool", [
    ((3, 5), (8, 12), (2, 2)),        # 2-D, rows of whole 16-byte pieces: the exact-tiling kernel
    ((2,), (6, 4, 8), (2, 2, 2)),     # 3-D
    ((7,), (2, 2, 4), (2, 2, 2)),     # a single window slab per volume
    ((4,), (10, 6), (2, 2)),          # float32 rows of 4k + 2 columns: pieces of 8 bytes
    ((3, 2), (14, 14), (2, 2)),
    ((2,), (4, 6, 10), (2, 2, 2)),
    ((1,), (2, 2), (2, 2)),           # one window in all
])
def test_pool_windows_that_tile_the_input_exactly(pools, dtype, lead, X, pool):
    """Stride == pool extent and X == G * P: the kernels that work straight from global
    memory.  Ties, NaNs, -0.0 gradients and the float64 dx of a float32 input included."""
    rng = np.random.default_rng(350 + len(X) + X[-1])
    for trial in range(4):
        if trial == 0:
            x = rng.standard_normal((*lead, *X)).astype(dtype)
        else:
            x = rng.integers(0, 3, (*lead, *X)).astype(dtype)  # ties in almost every window
        if trial == 2:
            x[rng.random(x.shape) < 0.1] = np.nan
        out_shape = (*lead, *(xk // pk for xk, pk in zip(X, pool)))
        g = (rng.standard_normal(out_shape) * 10.0 ** rng.integers(-6, 6, out_shape)).astype(dtype)
        g[rng.random(out_shape) < 0.2] = -0.0
        want_out = ora.pool_forward(x, pool, pool, validate=False)
        want_dx = ora.pool_backward(x, g, pool, pool)  # float64
        assert np.array_equal(bits(pools.pool_fwd(x, pool, pool)), bits(want_out))
        assert np.array_equal(bits(pools.pool_bwd(x, g, pool, pool, dx_dtype=np.float64)), bits(want_dx))
        assert np.array_equal(bits(pools.pool_bwd(x, g, pool, pool)), bits(want_dx.astype(dtype)))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("X,pool,stride", [((7, 9001), (3, 3), (2, 2)), ((2, 5, 7000), (2, 3, 2), (1, 2, 3)),
                                           ((7, 70, 70), (2, 3, 3), (1, 2, 2)), ((5, 9000), (4, 2), (1, 1))])
def test_pool_rows_too_long_for_the_staged_kernels(pools, dtype, X, pool, stride):
    """One row of windows with its halo exceeds the LDS budget: the kernels that work
    element by element from global memory take over."""
    rng = np.random.default_rng(360 + len(X))
    x = rng.integers(0, 5, (3, *X)).astype(dtype)
    out_shape = (3, *(((xk - pk) // sk + 1) for xk, pk, sk in zip(X, pool, stride)))
    g = (rng.standard_normal(out_shape) * 10.0 ** rng.integers(-6, 6, out_shape)).astype(dtype)
    want_dx = ora.pool_backward(x, g, pool, stride)
    assert np.array_equal(bits(pools.pool_fwd(x, pool, stride)), bits(ora.pool_forward(x, pool, stride, validate=False)))
    assert np.array_equal(bits(pools.pool_bwd(x, g, pool, stride, dx_dtype=np.float64)), bits(want_dx))
    assert np.array_equal(bits(pools.pool_bwd(x, g, pool, stride)), bits(want_dx.astype(dtype)))


def test_pool_window_of_256_positions_fills_the_argmax_byte(pools):
    rng = np.random.default_rng(361)
    x = rng.integers(0, 50, (2, 20, 19)).astype(np.float64)
    g = rng.standard_normal((2, 5, 4))
    assert np.array_equal(pools.pool_fwd(x, (16, 16), 1), ora.pool_forward(x, (16, 16), 1))
    assert np.array_equal(bits(pools.pool_bwd(x, g, (16, 16), 1)), bits(ora.pool_backward(x, g, (16, 16), 1)))


def test_pool_order_of_summation_and_signed_zero(pools):
    x = np.array([[0.0, 0.0, 9.0, 0.0, 0.0]])
    for g in ([1e16, 1.0, -1e16], [1e16, -1e16, 1.0], [-0.0, -0.0, -0.0]):
        g = np.array([g])
        dx = pools.pool_bwd(x, g, (3,), (1,))
        assert np.array_equal(bits(dx), bits(ora.pool_backward(x, g, (3,), (1,))))
    dx = pools.pool_bwd(np.array([[1.0, 0.0]]), np.array([[-0.0]]), (2,), (2,))
    assert not np.signbit(dx).any()


def test_pool_nan_first_nan_wins(pools):
    x = np.array([[1.0, np.nan, 5.0, np.nan, 2.0, 3.0]])
    out = pools.pool_fwd(x, (4,), (1,))
    want = ora.pool_forward(x, (4,), (1,))
    assert np.array_equal(np.isnan(out), np.isnan(want)) and np.isnan(out).all()
    g = np.array([[2.0, 3.0, 5.0]])
    assert np.array_equal(pools.pool_bwd(x, g, (4,), (1,)), ora.pool_backward(x, g, (4,), (1,)))


@pytest.mark.parametrize("ties", [False, True])
def test_pool_config2_literal_full_size(pools, ties):
    # x (64,64,56,56) f64, pool 3x3 stride 2, floor placement -> (64,64,27,27);
    # the reference's validator rejects it ((56-3)/2+1 = 27.5), its window helper floors
    rng = np.random.default_rng(1002)
    shape = (64, 64, 56, 56)
    x = rng.integers(0, 8, shape).astype(np.float64) if ties else rng.standard_normal(shape)
    g = rng.standard_normal((64, 64, 27, 27))
    out = pools.pool_fwd(x, (3, 3), 2)
    dx = pools.pool_bwd(x, g, (3, 3), 2)
    want_out, want_dx = direct.pool(x, g, (3, 3), (2, 2))
    assert np.array_equal(bits(out), bits(want_out))
    assert np.array_equal(bits(dx), bits(want_dx))
    assert not dx[..., 55, :].any() and not dx[..., :, 55].any()  # never covered by a window
    # the NumPy restatement of the reference agrees on a slice it finishes quickly
    sl = slice(0, 4)
    assert np.array_equal(bits(out[sl]), bits(ora.pool_forward(x[sl], (3, 3), 2, validate=False)))
    assert np.array_equal(bits(dx[sl]), bits(ora.pool_backward(x[sl], g[sl], (3, 3), 2)))


@pytest.mark.parametrize("ties", [False, True])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_pool_config2_valid_full_size(pools, ties, dtype):
    # the neighbour of config 2 that the reference accepts: x (64,64,55,55), pool 3x3 stride 2 ->
    # (64,64,27,27) exactly; rows of 55 elements start on no 16-byte boundary
    rng = np.random.default_rng(1002)
    shape = (64, 64, 55, 55)
    x = (rng.integers(0, 8, shape) if ties else rng.standard_normal(shape)).astype(dtype)
    g = rng.standard_normal((64, 64, 27, 27)).astype(dtype)
    out = pools.pool_fwd(x, (3, 3), 2)
    dx = pools.pool_bwd(x, g, (3, 3), 2)
    dx64 = pools.pool_bwd(x, g, (3, 3), 2, dx_dtype=np.float64)
    want_out, want_dx = direct.pool(x, g, (3, 3), (2, 2))
    assert np.array_equal(bits(out), bits(want_out))
    assert np.array_equal(bits(dx64), bits(want_dx))
    assert np.array_equal(bits(dx), bits(want_dx.astype(dtype)))
    sl = slice(0, 4)
    assert np.array_equal(bits(out[sl]), bits(ora.pool_forward(x[sl], (3, 3), 2)))
    assert np.array_equal(bits(dx64[sl]), bits(ora.pool_backward(x[sl], g[sl], (3, 3), 2)))


def test_pool_config5_shape_full_size(pools):
    rng = np.random.default_rng(1006)
    x = rng.standard_normal((8, 32, 32, 64, 64)).astype(np.float32)
    g = rng.standard_normal((8, 32, 16, 32, 32)).astype(np.float32)
    out = pools.pool_fwd(x, (2, 2, 2), 2)
    dx = pools.pool_bwd(x, g, (2, 2, 2), 2)
    want_out, want_dx = direct.pool(x, g, (2, 2, 2), (2, 2, 2))
    assert np.array_equal(bits(out), bits(want_out))
    assert np.array_equal(bits(dx), bits(want_dx.astype(np.float32)))


# ----------------------------------------------------------------------------- convolution
def test_conv_reference_known_answers(abi, kats):
    for dtype in (np.float64, np.float32):
        for case in kats["conv"]:
            x, w = np.array(case["x"], dtype=dtype), np.array(case["w"], dtype=dtype)
            conf = (tuple(case["stride"]), tuple(case["padding"]), tuple(case["dilation"]))
            out = abi.conv_fwd(x, w, *conf)
            assert np.array_equal(out, np.array(case["out"], dtype=dtype)), case["source"]
            if "dx_of_ones" in case:
                g = np.ones_like(out)
                assert np.array_equal(abi.conv_dgrad(g, x.shape, w, *conf), np.array(case["dx_of_ones"], dtype=dtype))
                assert np.array_equal(abi.conv_wgrad(g, x, w.shape, *conf), np.array(case["dw_of_ones"], dtype=dtype))


def _random_case(rng, m, big):
    hi = 40 if big else 6
    N = int(rng.integers(1, 4))
    C = int(rng.integers(1, hi))
    F = int(rng.integers(1, hi))
    taps = tuple(int(v) for v in rng.integers(1, 4, m))
    dil = tuple(int(v) for v in rng.integers(1, 3, m))
    stride = tuple(int(v) for v in rng.integers(1, 4, m))
    pad = tuple(int(v) for v in rng.integers(0, 3, m))
    grid = tuple(int(v) for v in rng.integers(1, 12 if m < 3 else 6, m))
    extra = tuple(int(v) for v in rng.integers(0, 2, m))  # rows the floor rule never uses
    X = tuple(
        (g - 1) * s + (t - 1) * d + 1 - 2 * p + (e if e < s else 0)
        for g, s, t, d, p, e in zip(grid, stride, taps, dil, pad, extra)
    )
    if any(v < 1 for v in X):
        return None
    return (N, C, *X), (F, C, *taps), stride, pad, dil


@pytest.fixture(params=["small problems planned as such", "planned like large ones"])
def plan_mode(request, monkeypatch):
    """A convolution of a few microseconds is planned for few launches (table-driven kernels
    that read the filter bank in place); MYGRAD_HIP_TINY=0 plans it like a large one, which
    is how shapes this small reach the tap-major kernels' edge cases."""
    if request.param == "planned like large ones":
        monkeypatch.setenv("MYGRAD_HIP_TINY", "0")
    return request.param


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("m", [1, 2, 3])
@pytest.mark.parametrize("big", [False, True])
def test_conv_random_cases_vs_oracle(abi, dtype, m, big, plan_mode):
    rng = np.random.default_rng(400 + 10 * m + big)
    tol = TOL[np.dtype(dtype)]
    done = 0
    while done < 10:
        case = _random_case(rng, m, big)
        if case is None:
            continue
        x_shape, w_shape, s, p, d = case
        print("conv case", np.dtype(dtype).name, x_shape, w_shape, s, p, d, flush=True)
        x = rng.standard_normal(x_shape).astype(dtype)
        w = rng.standard_normal(w_shape).astype(dtype)
        want_out = direct.conv_forward(x, w, s, p, d)
        g = rng.standard_normal(want_out.shape).astype(dtype)
        out = abi.conv_fwd(x, w, s, p, d)
        assert out.shape == want_out.shape and out.dtype == dtype
        assert rel_err(out, want_out) <= tol
        assert rel_err(abi.conv_dgrad(g, x_shape, w, s, p, d), direct.conv_backward_x(g, x_shape, w, s, p, d)) <= tol
        assert rel_err(abi.conv_wgrad(g, x, w_shape, s, p, d), direct.conv_backward_w(g, x, w_shape, s, p, d)) <= tol
        done += 1


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("m", [1, 2, 3])
def test_conv_channel_counts_that_take_the_tap_major_kernels(abi, dtype, m, plan_mode):
    # channel / filter counts that are multiples of the K tile (8 or 16) select the
    # tap-major kernels; mix them with counts that do not, strides, dilation, padding
    rng = np.random.default_rng(500 + m)
    tol = TOL[np.dtype(dtype)]
    done = 0
    while done < 14:
        C = int(rng.choice([8, 16, 32, 48, 64]))
        F = int(rng.choice([8, 16, 24, 32, 64, 80, 128, 144]))
        N = int(rng.integers(1, 4))
        taps = tuple(int(v) for v in rng.integers(1, 4, m))
        dil = tuple(int(v) for v in rng.integers(1, 3, m))
        stride = tuple(int(v) for v in rng.integers(1, 4, m))
        pad = tuple(int(v) for v in rng.integers(0, 3, m))
        grid = tuple(int(v) for v in rng.integers(1, [40, 14, 7][m - 1], m))
        extra = tuple(int(v) for v in rng.integers(0, 2, m))
        X = tuple(
            (g - 1) * s + (t - 1) * d + 1 - 2 * p + (e if e < s else 0)
            for g, s, t, d, p, e in zip(grid, stride, taps, dil, pad, extra)
        )
        if any(v < 1 for v in X):
            continue
        x_shape, w_shape = (N, C, *X), (F, C, *taps)
        print("tap-major case", np.dtype(dtype).name, x_shape, w_shape, stride, pad, dil, flush=True)
        x = rng.standard_normal(x_shape).astype(dtype)
        w = rng.standard_normal(w_shape).astype(dtype)
        want_out = direct.conv_forward(x, w, stride, pad, dil)
        g = rng.standard_normal(want_out.shape).astype(dtype)
        assert rel_err(abi.conv_fwd(x, w, stride, pad, dil), want_out) <= tol
        assert rel_err(abi.conv_dgrad(g, x_shape, w, stride, pad, dil),
                       direct.conv_backward_x(g, x_shape, w, stride, pad, dil)) <= tol
        assert rel_err(abi.conv_wgrad(g, x, w_shape, stride, pad, dil),
                       direct.conv_backward_w(g, x, w_shape, stride, pad, dil)) <= tol
        done += 1


# Stride 2 along the last axis (float32, filter count a multiple of 16): every tile of the data
# gradient computes all 2 / 4 stride phases of its patch and writes them interleaved.  Even and
# odd extents (vector and element-wise stores, phases with fewer positions than the coarse grid),
# 1, 2 and 3 convolved axes, channel counts for every fused tile shape (16 .. 128 rows), filters
# with taps that some phases never see (1x1: three of four phases are all zero), dilation, and
# enough positions for persistent blocks, tail tiles and K slices.
FUSED_PHASE_CASES = [
    ((4, 64, 28, 28), (32, 64, 3, 3), (2, 2), (1, 1), (1, 1)),
    ((3, 128, 27, 27), (48, 128, 3, 3), (2, 2), (1, 1), (1, 1)),
    ((2, 32, 30, 36), (16, 32, 1, 1), (2, 2), (0, 0), (1, 1)),
    ((5, 16, 19, 24), (64, 16, 5, 3), (2, 2), (2, 1), (1, 2)),
    ((2, 48, 40, 44), (32, 48, 2, 2), (1, 2), (0, 1), (1, 1)),
    ((3, 64, 130), (16, 64, 7), (2,), (3,), (1,)),
    ((2, 24, 9, 16, 20), (32, 24, 3, 3, 3), (1, 2, 2), (1, 1, 1), (1, 1, 1)),
    ((40, 128, 28, 28), (256, 128, 3, 3), (2, 2), (1, 1), (1, 1)),
    ((2, 8, 12, 10), (16, 8, 3, 3), (2, 2), (0, 0), (1, 1)),
    # exact window grids under stride 2 (odd extents): rows of dx start on no 16-byte boundary; an even
    # and an odd number of coarse positions per row (pairs of positions / single positions per store)
    ((3, 64, 13, 13), (32, 64, 3, 3), (2, 2), (1, 1), (1, 1)),
    ((2, 32, 55, 55), (64, 32, 3, 3), (2, 2), (1, 1), (1, 1)),
    ((2, 128, 9, 27), (16, 128, 3, 3), (1, 2), (1, 1), (1, 1)),
    ((2, 16, 5, 7, 11), (32, 16, 3, 3, 3), (1, 2, 2), (1, 1, 1), (1, 1, 1)),
    ((2, 64, 15, 15), (32, 64, 1, 1), (2, 2), (0, 0), (1, 1)),
]


@pytest.mark.parametrize("rows", ["short rows fused too", "short rows phase by phase"])
@pytest.mark.parametrize("case", range(len(FUSED_PHASE_CASES)))
def test_conv_dgrad_with_fused_stride_phases(abi, case, plan_mode, rows, monkeypatch):
    # four phases of rows shorter than 20 elements are planned phase by phase unless told otherwise
    if rows == "short rows fused too":
        monkeypatch.setenv("MYGRAD_HIP_FUSE_MIN_ROW", "0")
    x_shape, w_shape, s, p, d = FUSED_PHASE_CASES[case]
    rng = np.random.default_rng(900 + case)
    w = (rng.standard_normal(w_shape) / np.sqrt(np.prod(w_shape[1:]))).astype(np.float32)
    grid = tuple((x + 2 * pp - ((t - 1) * dd + 1)) // ss + 1 for x, t, ss, pp, dd in zip(x_shape[2:], w_shape[2:], s, p, d))
    g = rng.standard_normal((x_shape[0], w_shape[0], *grid)).astype(np.float32)
    dx = abi.conv_dgrad(g, x_shape, w, s, p, d)
    assert rel_err(dx, direct.conv_backward_x(g, x_shape, w, s, p, d)) <= 2e-4
    assert np.array_equal(dx, abi.conv_dgrad(g, x_shape, w, s, p, d))  # no atomics: run-to-run identical
    # dx of an all-ones gradient counts, per input element, the windows that reach it: exact
    # in float32 with a filter of ones, which isolates the routing from the rounding
    ones_w = np.ones(w_shape, dtype=np.float32)
    ones_g = np.ones_like(g)
    assert np.array_equal(abi.conv_dgrad(ones_g, x_shape, ones_w, s, p, d),
                          direct.conv_backward_x(ones_g, x_shape, ones_w, s, p, d).astype(np.float32))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("x_shape,w_shape,s,p,d", [
    ((5, 64, 7, 7), (64, 64, 3, 3), (1, 1), (1, 1), (1, 1)),       # 49 positions per sample
    ((3, 64, 27, 27), (128, 64, 3, 3), (1, 1), (1, 1), (1, 1)),    # 729
    ((2, 48, 5, 9, 3), (64, 48, 3, 3, 1), (1, 1, 1), (1, 1, 0), (1, 1, 1)),
    ((7, 128, 13), (64, 128, 5), (1,), (2,), (1,)),
    ((4, 64, 30, 31), (64, 64, 3, 3), (2, 2), (1, 1), (1, 1)),     # forward only: a 15 x 15 grid
])
def test_conv_samples_that_are_no_whole_16_byte_pieces(abi, dtype, x_shape, w_shape, s, p, d, monkeypatch):
    """An odd number of positions per sample: a lane's positions are adjacent in the result but
    not 16-byte aligned, and the last lane of a sample holds positions of two samples."""
    monkeypatch.setenv("MYGRAD_HIP_TINY", "0")
    rng = np.random.default_rng(1450 + x_shape[-1])
    tol = TOL[np.dtype(dtype)]
    x = rng.standard_normal(x_shape).astype(dtype)
    w = (rng.standard_normal(w_shape) / np.sqrt(np.prod(w_shape[1:]))).astype(dtype)
    want = direct.conv_forward(x, w, s, p, d)
    g = rng.standard_normal(want.shape).astype(dtype)
    assert rel_err(abi.conv_fwd(x, w, s, p, d), want) <= tol
    assert rel_err(abi.conv_dgrad(g, x_shape, w, s, p, d), direct.conv_backward_x(g, x_shape, w, s, p, d)) <= tol
    assert rel_err(abi.conv_wgrad(g, x, w_shape, s, p, d), direct.conv_backward_w(g, x, w_shape, s, p, d)) <= tol
    # exact with ones: an element stored to the wrong place changes a count
    ones_x, ones_w = np.ones(x_shape, dtype), np.ones(w_shape, dtype)
    assert np.array_equal(abi.conv_fwd(ones_x, ones_w, s, p, d), direct.conv_forward(ones_x, ones_w, s, p, d).astype(dtype))
    ones_g = np.ones_like(g)
    assert np.array_equal(abi.conv_dgrad(ones_g, x_shape, ones_w, s, p, d),
                          direct.conv_backward_x(ones_g, x_shape, ones_w, s, p, d).astype(dtype))


# Few channels (filters, in the forward pass), a 3-tap "same" last axis whose rows are a power of
# two up to 64 long (float32, the other count a multiple of 16): the data gradient and the forward
# pass compute the three taps of the last axis as separate rows and add them, shifted, in the epilogue.  1, 2 and 3 convolved axes,
# row lengths 4 .. 64, channel counts that do and do not fill the tile, other axes with padding,
# dilation and even tap counts, position counts that are no multiple of the tile.
FOLDED_TAP_CASES = [
    ((2, 16, 8, 64, 64), (32, 16, 3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    ((3, 16, 40, 32), (16, 16, 3, 3), (1, 1), (1, 1), (1, 1)),
    ((5, 8, 21, 16), (48, 8, 2, 3), (1, 1), (0, 1), (1, 1)),
    ((7, 5, 9, 8), (16, 5, 5, 3), (1, 1), (4, 1), (2, 1)),
    ((9, 12, 64), (32, 12, 3), (1,), (1,), (1,)),
    ((2, 3, 6, 10, 4), (16, 3, 1, 3, 3), (1, 1, 1), (0, 0, 1), (1, 1, 1)),
    ((1, 16, 33, 64), (64, 16, 1, 3), (1, 1), (0, 1), (1, 1)),
    ((2, 32, 16, 32), (16, 32, 3, 3), (1, 1), (1, 1), (1, 1)),       # 32 channels: 96-row tiles
    ((3, 24, 10, 16), (32, 24, 3, 3), (1, 1), (1, 1), (1, 1)),       # 24 channels in a 96-row tile
    ((2, 48, 12, 9, 32), (24, 48, 2, 3, 3), (2, 1, 1), (0, 2, 1), (1, 2, 1)),  # forward only folds (24 filters; stride on axis 0)
    # rows that are no power of two: padded to one (at most an eighth of padding), the padding never stored
    ((3, 16, 28, 28), (16, 16, 3, 3), (1, 1), (1, 1), (1, 1)),
    ((2, 8, 5, 14, 14), (32, 8, 3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    ((5, 16, 9, 7), (16, 16, 3, 3), (1, 1), (1, 1), (1, 1)),
    ((2, 16, 20, 56), (32, 16, 3, 3), (1, 1), (1, 1), (1, 1)),
    ((3, 10, 11, 30), (16, 10, 2, 3), (1, 1), (1, 1), (1, 1)),       # rows of 30: no whole 16-byte pieces, element-wise stores
    ((4, 16, 6, 15), (16, 16, 3, 3), (1, 1), (1, 1), (1, 1)),
    ((7, 32, 61), (32, 32, 3), (1,), (1,), (1,)),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", range(len(FOLDED_TAP_CASES)))
def test_conv_with_the_last_axis_taps_folded_into_rows(abi, case, dtype, monkeypatch):
    monkeypatch.setenv("MYGRAD_HIP_TINY", "0")  # small shapes: planned like large ones, or they take the table-driven kernel
    x_shape, w_shape, s, p, d = FOLDED_TAP_CASES[case]
    rng = np.random.default_rng(1300 + case)
    tol = TOL[np.dtype(dtype)]
    w = (rng.standard_normal(w_shape) / np.sqrt(np.prod(w_shape[1:]))).astype(dtype)
    grid = tuple((x + 2 * pp - ((t - 1) * dd + 1)) // ss + 1 for x, t, ss, pp, dd in zip(x_shape[2:], w_shape[2:], s, p, d))
    g = rng.standard_normal((x_shape[0], w_shape[0], *grid)).astype(dtype)
    dx = abi.conv_dgrad(g, x_shape, w, s, p, d)
    assert rel_err(dx, direct.conv_backward_x(g, x_shape, w, s, p, d)) <= tol
    assert np.array_equal(dx, abi.conv_dgrad(g, x_shape, w, s, p, d))
    # exact with ones: per input element, the number of (filter, tap) pairs that reach it -- a
    # shift in the wrong direction or a neighbour taken across a row end changes the counts
    ones_w = np.ones(w_shape, dtype=dtype)
    ones_g = np.ones_like(g)
    assert np.array_equal(abi.conv_dgrad(ones_g, x_shape, ones_w, s, p, d),
                          direct.conv_backward_x(ones_g, x_shape, ones_w, s, p, d).astype(dtype))
    # and with a filter that is not symmetric along the last axis (tap t2 weighs t2 + 1), so that
    # tap 0 and tap 2 cannot be swapped unnoticed
    ramp_w = np.ones(w_shape, dtype=dtype) * np.arange(1, w_shape[-1] + 1, dtype=dtype)
    assert np.array_equal(abi.conv_dgrad(ones_g, x_shape, ramp_w, s, p, d),
                          direct.conv_backward_x(ones_g, x_shape, ramp_w, s, p, d).astype(dtype))
    # the forward pass folds the same way when there are few filters (and channels in whole K tiles)
    x = rng.standard_normal(x_shape).astype(dtype)
    out = abi.conv_fwd(x, w, s, p, d)
    assert rel_err(out, direct.conv_forward(x, w, s, p, d)) <= tol
    assert np.array_equal(out, abi.conv_fwd(x, w, s, p, d))
    # exact: x counts along the last axis (small integers), ramp filter
    steps = np.broadcast_to(np.arange(x_shape[-1], dtype=dtype) % 5, x_shape).copy()
    assert np.array_equal(abi.conv_fwd(steps, ramp_w, s, p, d), direct.conv_forward(steps, ramp_w, s, p, d).astype(dtype))


# Channel counts that fill no K tile (the one or three channels of a first layer), on problems
# large enough not to be planned as tiny: the forward pass runs the tap-major kernel with K tiles
# made of rows of the gather table (the last tile padded with rows that lie outside every input).
FIRST_LAYER_CASES = [
    ((16, 3, 64, 64), (32, 3, 5, 5), (1, 1), (2, 2), (1, 1)),
    ((8, 3, 115, 115), (64, 3, 7, 7), (2, 2), (3, 3), (1, 1)),      # the stem's geometry, flooring placement
    ((32, 1, 28, 28), (20, 1, 5, 5), (1, 1), (0, 0), (1, 1)),       # one channel, 20 filters (padded packed rows)
    ((4, 5, 20, 24, 24), (16, 5, 3, 3, 3), (1, 2, 1), (1, 0, 1), (1, 1, 2)),
    ((64, 7, 500), (48, 7, 9), (3,), (4,), (2,)),
    ((64, 1, 28, 28), (64, 1, 5, 5), (1, 1), (0, 0), (1, 1)),       # 25 columns of dw: one 32-column tile
    ((16, 3, 48, 48), (128, 3, 7, 7), (1, 1), (3, 3), (1, 1)),      # 147 columns: two 80-column tiles, two row tiles
    # filter counts that fill no K tile either: the data gradient on table rows, the filter gradient
    # with a short last row tile
    ((256, 1, 28, 28), (20, 1, 5, 5), (1, 1), (0, 0), (1, 1)),
    ((256, 20, 12, 12), (10, 20, 5, 5), (1, 1), (0, 0), (1, 1)),
    ((32, 24, 41, 40), (20, 24, 3, 4), (2, 2), (1, 1), (1, 1)),     # four stride phases with different tap counts
    ((6, 16, 10, 18, 18), (35, 16, 3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    ((64, 40, 301), (19, 40, 7), (2,), (3,), (3,)),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", range(len(FIRST_LAYER_CASES)))
def test_conv_with_channel_or_filter_counts_that_fill_no_k_tile(abi, dtype, case):
    x_shape, w_shape, s, p, d = FIRST_LAYER_CASES[case]
    rng = np.random.default_rng(1500 + case)
    tol = TOL[np.dtype(dtype)]
    x = rng.standard_normal(x_shape).astype(dtype)
    w = (rng.standard_normal(w_shape) / np.sqrt(np.prod(w_shape[1:]))).astype(dtype)
    want = direct.conv_forward(x, w, s, p, d)
    out = abi.conv_fwd(x, w, s, p, d)
    assert rel_err(out, want) <= tol
    assert np.array_equal(out, abi.conv_fwd(x, w, s, p, d))
    # exact: small integers, every (channel, tap) weighted differently
    xi = rng.integers(-2, 3, x_shape).astype(dtype)
    wi = (np.arange(np.prod(w_shape[1:])).reshape(w_shape[1:]) % 7 - 3).astype(dtype) * np.ones(w_shape, dtype=dtype)
    assert np.array_equal(abi.conv_fwd(xi, wi, s, p, d), direct.conv_forward(xi, wi, s, p, d).astype(dtype))
    g = rng.standard_normal(want.shape).astype(dtype)
    assert rel_err(abi.conv_dgrad(g, x_shape, w, s, p, d), direct.conv_backward_x(g, x_shape, w, s, p, d)) <= tol
    assert rel_err(abi.conv_wgrad(g, x, w_shape, s, p, d), direct.conv_backward_w(g, x, w_shape, s, p, d)) <= tol
    # exact: gradients of small integers
    gi = rng.integers(-2, 3, want.shape).astype(dtype)
    assert np.array_equal(abi.conv_dgrad(gi, x_shape, wi, s, p, d), direct.conv_backward_x(gi, x_shape, wi, s, p, d).astype(dtype))
    assert np.array_equal(abi.conv_wgrad(gi, xi, w_shape, s, p, d), direct.conv_backward_w(gi, xi, w_shape, s, p, d).astype(dtype))


# Up to four channels in single precision, on enough positions to fill the device: the data
# gradient runs one position of the coarse grid ceil(X / stride) per lane on the 4x4x1 MFMA, all
# stride phases of the position at once (1, 2 or 4 of them).  Between them the cases cover every
# phase count, entries that fill their chunks of 16 / phases and ones that need padding or
# several channels per chunk, odd extents (phases with different numbers of positions, no paired
# stores), dilation, and one to three convolved axes.  float64 runs the other kernels.
THIN_ROW_CASES = [
    ((16, 3, 130, 130), (16, 3, 7, 7), (2, 2), (3, 3), (1, 1)),     # the stem's geometry (even extent, flooring placement): 4 phases, 16 entries
    ((16, 3, 131, 131), (8, 3, 7, 7), (2, 2), (3, 3), (1, 1)),      # odd extents: the phases differ in size
    ((64, 3, 64, 64), (32, 3, 5, 5), (1, 1), (2, 2), (1, 1)),       # one phase, 25 entries, two filters per chunk step
    ((64, 1, 128, 128), (10, 1, 3, 3), (1, 1), (1, 1), (1, 1)),     # one channel; 9 entries x 2 filters, padded
    ((16, 4, 96, 97), (16, 4, 3, 4), (1, 2), (1, 1), (1, 1)),       # two phases along the last axis
    ((16, 2, 140, 70), (24, 2, 5, 3), (2, 1), (2, 1), (1, 1)),      # two phases along the first axis: no paired stores
    ((64, 3, 64, 64), (32, 3, 3, 3), (1, 1), (2, 2), (2, 2)),       # dilation 2; 9 entries x 16 filters fill their chunks
    ((4, 3, 18, 64, 64), (12, 3, 3, 3, 3), (1, 2, 2), (1, 1, 1), (1, 1, 1)),  # three axes, four phases
    ((64, 2, 2100), (48, 2, 9), (2,), (4,), (1,)),                  # one axis, two phases
    ((64, 3, 128, 128), (16, 3, 2, 2), (2, 2), (0, 0), (1, 1)),     # window = stride: every phase has one tap
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", range(len(THIN_ROW_CASES)))
def test_data_gradient_with_up_to_four_channels(abi, dtype, case):
    x_shape, w_shape, s, p, d = THIN_ROW_CASES[case]
    rng = np.random.default_rng(2300 + case)
    tol = TOL[np.dtype(dtype)]
    w = (rng.standard_normal(w_shape) / np.sqrt(np.prod(w_shape[1:]))).astype(dtype)
    grid = direct.conv_forward(np.zeros(x_shape, dtype=dtype), w, s, p, d).shape
    g = rng.standard_normal(grid).astype(dtype)
    got = abi.conv_dgrad(g, x_shape, w, s, p, d)
    assert rel_err(got, direct.conv_backward_x(g, x_shape, w, s, p, d)) <= tol
    assert np.array_equal(got, abi.conv_dgrad(g, x_shape, w, s, p, d))
    # exact: small integers, every (filter, channel, tap) weighted differently
    gi = rng.integers(-2, 3, grid).astype(dtype)
    wi = (np.arange(np.prod(w_shape)).reshape(w_shape) % 11 - 5).astype(dtype)
    assert np.array_equal(abi.conv_dgrad(gi, x_shape, wi, s, p, d), direct.conv_backward_x(gi, x_shape, wi, s, p, d).astype(dtype))
    if dtype == np.float32:
        # MYGRAD_HIP_THIN=0 plans the same problem on the 16-row tiles: same bar
        os.environ["MYGRAD_HIP_THIN"] = "0"
        try:
            other = abi.conv_dgrad(g, x_shape, w, s, p, d)
        finally:
            del os.environ["MYGRAD_HIP_THIN"]
        assert rel_err(other, direct.conv_backward_x(g, x_shape, w, s, p, d)) <= tol


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("x_shape,w_shape,s,p,d", [
    ((8, 3, 101, 100), (64, 3, 7, 7), (2, 2), (3, 3), (1, 1)),     # too few positions for the kernel above in float32
    ((6, 4, 75, 81), (32, 4, 5, 5), (2, 2), (2, 2), (1, 1)),       # sixteen rows: four channels x four phases, odd extents
    ((4, 8, 90, 64), (48, 8, 3, 4), (2, 1), (1, 2), (1, 1)),       # two phases along the first axis only: no paired stores
    ((3, 2, 30, 41, 44), (16, 2, 3, 3, 3), (1, 2, 2), (1, 1, 1), (1, 1, 1)),
    ((16, 5, 4000), (32, 5, 9), (2,), (4,), (2,)),                 # dilation 2 under stride 2: one phase has no tap at all
])
def test_data_gradient_with_the_stride_phases_as_rows(abi, dtype, x_shape, w_shape, s, p, d):
    """A few channels under a stride where the one-position-per-lane kernel does not apply (double
    precision, or too few positions): the rows of the GEMM are (channel, stride phase) over the
    coarse grid.  MYGRAD_HIP_PHASE_ROWS=0 plans the same problem phase by phase: same bar."""
    rng = np.random.default_rng(2500 + x_shape[-1])
    tol = TOL[np.dtype(dtype)]
    w = (rng.standard_normal(w_shape) / np.sqrt(np.prod(w_shape[1:]))).astype(dtype)
    grid = direct.conv_forward(np.zeros(x_shape, dtype=dtype), w, s, p, d).shape
    g = rng.standard_normal(grid).astype(dtype)
    want = direct.conv_backward_x(g, x_shape, w, s, p, d)
    got = abi.conv_dgrad(g, x_shape, w, s, p, d)
    assert rel_err(got, want) <= tol
    assert np.array_equal(got, abi.conv_dgrad(g, x_shape, w, s, p, d))
    gi = rng.integers(-2, 3, grid).astype(dtype)
    wi = (np.arange(np.prod(w_shape)).reshape(w_shape) % 11 - 5).astype(dtype)
    assert np.array_equal(abi.conv_dgrad(gi, x_shape, wi, s, p, d), direct.conv_backward_x(gi, x_shape, wi, s, p, d).astype(dtype))
    os.environ["MYGRAD_HIP_PHASE_ROWS"] = "0"
    try:
        other = abi.conv_dgrad(g, x_shape, w, s, p, d)
    finally:
        del os.environ["MYGRAD_HIP_PHASE_ROWS"]
    assert rel_err(other, want) <= tol


# Every tile shape of the forward / data-gradient kernels, forced in turn (the planner would take
# one or two of them for any given problem): rows x positions, and for the data gradient under a
# stride the shapes of its fused stride phases.
ALL_TILES = ["128,128", "128,64", "64,256", "64,128", "32,256", "32,128", "16,256", "64,64"]
TILE_PROBLEMS = [
    # (x, w, stride, padding, dilation): odd extents, so that row ends and sample ends fall inside tiles
    ((3, 32, 29, 27), (160, 32, 3, 3), (1, 1), (1, 1), (1, 1)),       # 160 rows: one and a quarter tiles of 128
    ((2, 48, 31, 33), (48, 48, 3, 3), (2, 2), (1, 1), (1, 1)),        # stride 2 both ways: four fused phases
    ((2, 32, 20, 45), (64, 32, 3, 5), (1, 2), (1, 2), (1, 1)),        # stride 2 along the last axis only: two fused phases
    ((2, 16, 9, 17, 19), (32, 16, 3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),  # three axes; folded taps where the tile allows
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("tile", ALL_TILES)
@pytest.mark.parametrize("problem", range(len(TILE_PROBLEMS)))
def test_every_tile_shape_of_the_gather_gemm(abi, monkeypatch, problem, tile, dtype):
    from mygrad_amd import _hip

    monkeypatch.setenv("MYGRAD_HIP_TINY", "0")
    monkeypatch.setenv("MYGRAD_HIP_TILE", tile)
    monkeypatch.setenv("MYGRAD_HIP_FUSE_MIN_ROW", "0")
    x_shape, w_shape, s, p, d = TILE_PROBLEMS[problem]
    rng = np.random.default_rng(2700 + problem)
    tol = TOL[np.dtype(dtype)]
    x = rng.standard_normal(x_shape).astype(dtype)
    w = (rng.standard_normal(w_shape) / np.sqrt(np.prod(w_shape[1:]))).astype(dtype)
    want = direct.conv_forward(x, w, s, p, d)
    got = abi.conv_fwd(x, w, s, p, d)
    print("forward:", _hip.last_plan(), flush=True)
    assert rel_err(got, want) <= tol
    g = rng.standard_normal(want.shape).astype(dtype)
    dx = abi.conv_dgrad(g, x_shape, w, s, p, d)
    print("data gradient:", _hip.last_plan(), flush=True)
    assert rel_err(dx, direct.conv_backward_x(g, x_shape, w, s, p, d)) <= tol
    # small integers: every sum is exact whatever the tile and however its K tiles are shared out
    xi = rng.integers(-3, 4, x_shape).astype(dtype)
    wi = rng.integers(-2, 3, w_shape).astype(dtype)
    gi = rng.integers(-2, 3, want.shape).astype(dtype)
    assert np.array_equal(abi.conv_fwd(xi, wi, s, p, d), direct.conv_forward(xi, wi, s, p, d).astype(dtype))
    assert np.array_equal(abi.conv_dgrad(gi, x_shape, wi, s, p, d), direct.conv_backward_x(gi, x_shape, wi, s, p, d).astype(dtype))


@pytest.mark.parametrize("x_shape,w_shape,row_tiles", [
    ((16, 32, 32, 32), (512, 32, 3, 3), 4),
    ((8, 16, 32, 32), (1024, 16, 3, 3), 8),
])
def test_row_tiles_of_a_position_block_on_one_xcd(abi, monkeypatch, x_shape, w_shape, row_tiles):
    """As many tiles as the device has block slots, 4 or 8 row tiles per position block: the blocks
    start on the tiles in chunks per XCD (every tile must still be computed exactly once), and with
    MYGRAD_HIP_XCD_CHUNK=0 on the tile of their own number; same results bit for bit."""
    from mygrad_amd import _hip

    monkeypatch.setenv("MYGRAD_HIP_TILE", "128,128,2")
    rng = np.random.default_rng(2900 + row_tiles)
    x = rng.standard_normal(x_shape).astype(np.float32)
    w = (rng.standard_normal(w_shape) / np.sqrt(np.prod(w_shape[1:]))).astype(np.float32)
    got = abi.conv_fwd(x, w, 1, 1, 1)
    assert f"x {row_tiles} row tiles" in _hip.last_plan() and "tile 128x128" in _hip.last_plan()
    assert rel_err(got, direct.conv_forward(x, w, (1, 1), (1, 1), (1, 1))) <= 2e-4
    monkeypatch.setenv("MYGRAD_HIP_XCD_CHUNK", "0")  # read at every launch
    assert np.array_equal(bits(got), bits(abi.conv_fwd(x, w, 1, 1, 1)))


WGRAD_TILES = ["128,128", "64,64", "32,128", "32,64", "16,64"]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("tile", WGRAD_TILES)
@pytest.mark.parametrize("x_shape,w_shape,s,p,d", [
    ((3, 32, 29, 27), (128, 32, 3, 3), (1, 1), (1, 1), (1, 1)),   # 288 columns: tiles of 128 overhang
    ((2, 48, 31, 33), (64, 48, 3, 3), (2, 2), (1, 1), (1, 1)),    # rows of grad that are no whole 16-byte pieces
])
def test_every_tile_shape_of_the_filter_gradient(abi, monkeypatch, x_shape, w_shape, s, p, d, tile, dtype):
    from mygrad_amd import _hip

    monkeypatch.setenv("MYGRAD_HIP_TINY", "0")
    monkeypatch.setenv("MYGRAD_HIP_WGRAD_TILE", tile)
    rng = np.random.default_rng(2800 + x_shape[-1])
    x = rng.standard_normal(x_shape).astype(dtype)
    grid = direct.conv_forward(x, np.zeros(w_shape, dtype=dtype), s, p, d).shape
    g = rng.standard_normal(grid).astype(dtype)
    got = abi.conv_wgrad(g, x, w_shape, s, p, d)
    print("filter gradient:", _hip.last_plan(), flush=True)
    assert rel_err(got, direct.conv_backward_w(g, x, w_shape, s, p, d)) <= TOL[np.dtype(dtype)]
    xi = rng.integers(-3, 4, x_shape).astype(dtype)
    gi = rng.integers(-2, 3, grid).astype(dtype)
    assert np.array_equal(abi.conv_wgrad(gi, xi, w_shape, s, p, d), direct.conv_backward_w(gi, xi, w_shape, s, p, d).astype(dtype))


# The filter gradient's K index is the position: the single-precision tap-major kernel reads, per
# position, a row of a table (window origin in x, which taps exist, what the sample adds to the
# offset into grad) instead of dividing the position into coordinates for every K tile.
POS_TABLE_CASES = [
    ((6, 16, 23, 23), (32, 16, 3, 3), (1, 1), (1, 1), (1, 1)),         # rows of grad that are no whole 16-byte pieces
    ((4, 32, 20, 24), (16, 32, 3, 3), (2, 2), (1, 1), (1, 1)),         # stride: taps missing on one side only
    ((3, 16, 31, 36), (64, 16, 7, 7), (2, 1), (3, 3), (1, 1)),         # 49 taps: both words of the tap mask
    ((2, 16, 9, 20, 20), (32, 16, 3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),  # 27 taps, padding on three axes
    ((5, 48, 40, 40), (128, 48, 5, 5), (1, 1), (4, 4), (2, 2)),        # dilation; wide tiles, several column groups per thread
    ((2, 16, 12, 12), (16, 16, 3, 3), (1, 1), (2, 2), (1, 1)),         # padding wider than a tap step; one short K tile per split
    # channels that fill no group of 16 columns: one table row per column, its tap looked up in the position's mask
    ((8, 3, 45, 45), (64, 3, 7, 7), (2, 2), (3, 3), (1, 1)),           # 147 columns in two tiles of 80
    ((6, 5, 22, 26), (24, 5, 3, 3), (1, 1), (1, 1), (1, 1)),           # a short last row tile; rows of grad that are no whole pieces
    ((4, 20, 15, 15), (10, 20, 5, 5), (1, 1), (0, 0), (1, 1)),         # no padding: every tap exists everywhere
]


@pytest.mark.parametrize("x_shape,w_shape,s,p,d", POS_TABLE_CASES)
def test_filter_gradient_with_and_without_the_position_table(abi, monkeypatch, x_shape, w_shape, s, p, d):
    monkeypatch.setenv("MYGRAD_HIP_TINY", "0")  # small shapes: planned like large ones, or they take the table-driven kernel
    rng = np.random.default_rng(2600 + x_shape[-1])
    x = rng.standard_normal(x_shape).astype(np.float32)
    grid = direct.conv_forward(x, np.zeros(w_shape, dtype=np.float32), s, p, d).shape
    g = rng.standard_normal(grid).astype(np.float32)
    want = direct.conv_backward_w(g, x, w_shape, s, p, d)
    got = abi.conv_wgrad(g, x, w_shape, s, p, d)
    from mygrad_amd import _hip

    assert "tap-major" in _hip.last_plan()
    assert rel_err(got, want) <= TOL[np.dtype(np.float32)]
    # small integers: every sum is exact, so the result is the definition's bit for bit
    xi = rng.integers(-3, 4, x_shape).astype(np.float32)
    gi = rng.integers(-2, 3, grid).astype(np.float32)
    assert np.array_equal(abi.conv_wgrad(gi, xi, w_shape, s, p, d), direct.conv_backward_w(gi, xi, w_shape, s, p, d).astype(np.float32))
    # the same kernel on its own position arithmetic adds the same terms in the same order
    monkeypatch.setenv("MYGRAD_HIP_POS_TABLE", "0")
    assert np.array_equal(bits(got), bits(abi.conv_wgrad(g, x, w_shape, s, p, d)))


# Up to four filters in single precision (a layer that ends in one map or in the three colours
# of an image), or a first layer (channels that fill no K tile): the forward pass on the same
# kernel, one output position per lane.
THIN_FILTER_CASES = [
    ((64, 16, 64, 64), (3, 16, 3, 3), (1, 1), (1, 1), (1, 1)),
    ((256, 64, 64, 64), (1, 64, 1, 1), (1, 1), (0, 0), (1, 1)),     # one tap: sixteen channels per chunk
    ((112, 8, 97, 97), (4, 8, 7, 7), (2, 2), (3, 3), (1, 1)),       # strided reads
    ((4, 6, 20, 64, 64), (2, 6, 3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    ((128, 48, 2048), (3, 48, 5), (1,), (4,), (2,)),
    ((64, 9, 64, 64), (4, 9, 5, 5), (1, 1), (2, 2), (1, 1)),        # 25 taps, 9 channels: one channel per group, chunks padded
    # a first layer with more than 64 filters: passes of 64 rows over the same positions
    ((128, 3, 64, 64), (96, 3, 4, 4), (2, 2), (1, 1), (1, 1)),      # a pass of 64 and one of 32
    ((64, 1, 64, 64), (130, 1, 3, 3), (1, 1), (1, 1), (1, 1)),      # three passes, two rows in the last
    # a first layer of 8, 16 and 32 filters: two, four and eight groups of four rows
    ((64, 3, 64, 64), (8, 3, 3, 3), (1, 1), (1, 1), (1, 1)),
    ((32, 3, 96, 96), (16, 3, 5, 5), (2, 2), (2, 2), (1, 1)),
    ((64, 2, 64, 64), (32, 2, 3, 3), (1, 1), (1, 1), (1, 1)),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", range(len(THIN_FILTER_CASES)))
def test_forward_pass_with_up_to_four_filters(abi, dtype, case):
    x_shape, w_shape, s, p, d = THIN_FILTER_CASES[case]
    rng = np.random.default_rng(2400 + case)
    tol = TOL[np.dtype(dtype)]
    x = rng.standard_normal(x_shape).astype(dtype)
    w = (rng.standard_normal(w_shape) / np.sqrt(np.prod(w_shape[1:]))).astype(dtype)
    got = abi.conv_fwd(x, w, s, p, d)
    assert rel_err(got, direct.conv_forward(x, w, s, p, d)) <= tol
    assert np.array_equal(got, abi.conv_fwd(x, w, s, p, d))
    xi = rng.integers(-2, 3, x_shape).astype(dtype)
    wi = (np.arange(np.prod(w_shape)).reshape(w_shape) % 11 - 5).astype(dtype)
    assert np.array_equal(abi.conv_fwd(xi, wi, s, p, d), direct.conv_forward(xi, wi, s, p, d).astype(dtype))
    if dtype == np.float32:
        os.environ["MYGRAD_HIP_THIN"] = "0"  # the same problem on the 16-row tiles: same bar
        try:
            other = abi.conv_fwd(x, w, s, p, d)
        finally:
            del os.environ["MYGRAD_HIP_THIN"]
        assert rel_err(other, direct.conv_forward(x, w, s, p, d)) <= tol


def _random_medium_case(rng, m):
    """A random problem of 0.12 - 3 GFLOP: large enough to be planned like the benchmark's
    layers (whichever family its channel and filter counts select), small enough for the oracle."""
    C = int(rng.choice([1, 3, 8, 16, 20, 32, 48, 64]))
    F = int(rng.choice([2, 4, 10, 16, 24, 32, 64, 96]))
    taps = tuple(int(v) for v in rng.integers(1, 6 if m < 3 else 4, m))
    dil = tuple(int(v) for v in rng.integers(1, 3, m))
    stride = tuple(int(v) for v in rng.integers(1, 4, m))
    pad = tuple(int(v) for v in rng.integers(0, 3, m))
    grid = tuple(int(v) for v in rng.integers(6, {1: 900, 2: 60, 3: 20}[m], m))
    X = tuple((g - 1) * s + (t - 1) * d + 1 - 2 * p + int(rng.integers(0, s)) for g, s, t, d, p in zip(grid, stride, taps, dil, pad))
    if any(v < 1 for v in X):
        return None
    per_sample = 2 * int(np.prod(grid)) * C * F * int(np.prod(taps))
    N = max(1, -(-150_000_000 // per_sample))
    if N > 512 or N * per_sample > 3_000_000_000 or N * max(C * int(np.prod(X)), F * int(np.prod(grid))) > 50_000_000:
        return None
    return (N, C, *X), (F, C, *taps), stride, pad, dil


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("m", [1, 2, 3])
def test_conv_random_problems_of_benchmark_size(abi, dtype, m):
    rng = np.random.default_rng(2700 + m)
    tol = TOL[np.dtype(dtype)]
    done = 0
    while done < 10:
        case = _random_medium_case(rng, m)
        if case is None:
            continue
        x_shape, w_shape, s, p, d = case
        print("medium case", np.dtype(dtype).name, x_shape, w_shape, s, p, d, flush=True)
        x = rng.standard_normal(x_shape).astype(dtype)
        w = (rng.standard_normal(w_shape) / np.sqrt(np.prod(w_shape[1:]))).astype(dtype)
        want = direct.conv_forward(x, w, s, p, d)
        g = rng.standard_normal(want.shape).astype(dtype)
        assert rel_err(abi.conv_fwd(x, w, s, p, d), want) <= tol
        assert rel_err(abi.conv_dgrad(g, x_shape, w, s, p, d), direct.conv_backward_x(g, x_shape, w, s, p, d)) <= tol
        assert rel_err(abi.conv_wgrad(g, x, w_shape, s, p, d), direct.conv_backward_w(g, x, w_shape, s, p, d)) <= tol
        done += 1


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("filters", [10, 16])
def test_conv_whose_windows_step_over_the_only_row(abi, dtype, filters):
    """An axis of one element, padded by one, under a one-element window with stride 2: the
    windows sit on the two padding rows and never on x.  The output is zero, dw is zero, and dx
    is zero because no stride phase has a tap (the data gradient's tables are empty) -- on a
    problem large enough to be planned like any other."""
    x_shape, w_shape, s, p, d = (64, 20, 1, 2048), (filters, 20, 1, 3), (2, 1), (1, 1), (1, 1)
    rng = np.random.default_rng(2600 + filters)
    x = rng.standard_normal(x_shape).astype(dtype)
    w = rng.standard_normal(w_shape).astype(dtype)
    out = abi.conv_fwd(x, w, s, p, d)
    assert out.shape == (64, filters, 2, 2048) and not out.any()
    g = rng.standard_normal(out.shape).astype(dtype)
    dx = abi.conv_dgrad(g, x_shape, w, s, p, d)
    assert dx.shape == x_shape and not dx.any()
    assert not direct.conv_backward_x(g, x_shape, w, s, p, d).any()
    dw = abi.conv_wgrad(g, x, w_shape, s, p, d)
    assert dw.shape == w_shape and not dw.any()


def _random_thin_case(rng, m, rows_are_channels):
    """A random problem with few rows (channels for the data gradient, filters for the forward
    pass) and enough positions for the one-position-per-lane kernel: strides of 1 or 2 (1, 2 or 4
    stride phases, or more: then the other kernels run), windows of 1 to 5, dilation, padding."""
    few = int(rng.integers(1, 5))
    many = int(rng.choice([8, 16, 20, 33]))
    C, F = (few, many) if rows_are_channels else (many, few)
    taps = tuple(int(v) for v in rng.integers(1, 6 if m < 3 else 4, m))
    dil = tuple(int(v) for v in rng.integers(1, 3, m))
    stride = tuple(int(v) for v in rng.integers(1, 3, m))
    pad = tuple(int(v) for v in rng.integers(0, 3, m))
    grid = tuple(int(v) for v in rng.integers(20, {1: 600, 2: 70, 3: 24}[m], m))
    X = tuple((g - 1) * s + (t - 1) * d + 1 - 2 * p + int(rng.integers(0, s)) for g, s, t, d, p in zip(grid, stride, taps, dil, pad))
    if any(v < 1 for v in X):
        return None
    coarse = int(np.prod([-(-v // s) for v, s in zip(X, stride)])) if rows_are_channels else int(np.prod(grid))
    # enough positions, and enough work not to be planned as a problem of a few microseconds
    N = max(-(-300000 // coarse), -(-120_000_000 // (2 * coarse * C * F * int(np.prod(taps)))))
    if N * max(C, F) * int(np.prod(X)) > 60_000_000:
        return None
    return (N, C, *X), (F, C, *taps), stride, pad, dil


@pytest.mark.parametrize("m", [1, 2, 3])
@pytest.mark.parametrize("which", ["data gradient, few channels", "forward, few filters"])
def test_random_problems_with_few_rows(abi, m, which):
    rows_are_channels = which.startswith("data")
    rng = np.random.default_rng(2500 + 10 * m + rows_are_channels)
    done = 0
    while done < 8:
        case = _random_thin_case(rng, m, rows_are_channels)
        if case is None:
            continue
        x_shape, w_shape, s, p, d = case
        print("thin case", which, x_shape, w_shape, s, p, d, flush=True)
        w = (rng.standard_normal(w_shape) / np.sqrt(np.prod(w_shape[1:]))).astype(np.float32)
        wi = (np.arange(np.prod(w_shape)).reshape(w_shape) % 11 - 5).astype(np.float32)
        if rows_are_channels:
            grid = direct.conv_forward(np.zeros(x_shape, dtype=np.float32), w, s, p, d).shape
            g = rng.standard_normal(grid).astype(np.float32)
            assert rel_err(abi.conv_dgrad(g, x_shape, w, s, p, d), direct.conv_backward_x(g, x_shape, w, s, p, d)) <= 2e-4
            gi = rng.integers(-2, 3, grid).astype(np.float32)
            assert np.array_equal(abi.conv_dgrad(gi, x_shape, wi, s, p, d), direct.conv_backward_x(gi, x_shape, wi, s, p, d).astype(np.float32))
        else:
            x = rng.standard_normal(x_shape).astype(np.float32)
            assert rel_err(abi.conv_fwd(x, w, s, p, d), direct.conv_forward(x, w, s, p, d)) <= 2e-4
            xi = rng.integers(-2, 3, x_shape).astype(np.float32)
            assert np.array_equal(abi.conv_fwd(xi, wi, s, p, d), direct.conv_forward(xi, wi, s, p, d).astype(np.float32))
        done += 1


# Shapes picked so that, between them, every tile shape and code path of the tap-major
# kernels runs: all gather-GEMM tiles (rows 16..128), persistent blocks that stream
# through several tiles and K slices, strided dgrad phases, filter counts that are not a
# multiple of four (padded packed rows), the 128x128 / 64x192 / 64x128 / 64x64 / 32x64 /
# 16x64 filter-gradient tiles, and an odd number of positions per sample (grad tile
# loaded element by element instead of 16 bytes per lane).
PADDED_CHANNEL_CASES = [
    # (x shape, w shape, stride, pad, dilation): large enough, channel / filter counts that are no
    # multiple of 16 but within a third of one: run on zero-padded copies by the tap-major kernels
    ((8, 24, 48, 48), (40, 24, 3, 3), (1, 1), (1, 1), (1, 1)),
    ((6, 40, 40, 40), (32, 40, 3, 3), (2, 2), (1, 1), (1, 1)),
    ((4, 32, 64, 64), (56, 32, 3, 3), (1, 1), (0, 0), (2, 2)),
    ((16, 100, 400), (72, 100, 5), (1,), (2,), (1,)),
    ((2, 24, 12, 20, 20), (24, 24, 3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
]


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("case", range(len(PADDED_CHANNEL_CASES)))
def test_conv_awkward_channel_counts_on_padded_copies(abi, dtype, case):
    x_shape, w_shape, s, p, d = PADDED_CHANNEL_CASES[case]
    rng = np.random.default_rng(700 + case)
    tol = TOL[np.dtype(dtype)]
    x = rng.standard_normal(x_shape).astype(dtype)
    w = (rng.standard_normal(w_shape) / np.sqrt(np.prod(w_shape[1:]))).astype(dtype)
    want_out = direct.conv_forward(x, w, s, p, d)
    g = rng.standard_normal(want_out.shape).astype(dtype)
    assert rel_err(abi.conv_fwd(x, w, s, p, d), want_out) <= tol
    assert rel_err(abi.conv_dgrad(g, x_shape, w, s, p, d), direct.conv_backward_x(g, x_shape, w, s, p, d)) <= tol
    assert rel_err(abi.conv_wgrad(g, x, w_shape, s, p, d), direct.conv_backward_w(g, x, w_shape, s, p, d)) <= tol


KERNEL_VARIANT_CASES = [
    # x shape, w shape, stride, padding, dilation
    ((8, 128, 28, 28), (128, 128, 3, 3), (1, 1), (1, 1), (1, 1)),   # 128-row tiles, wgrad 128x128
    ((32, 64, 28, 28), (64, 64, 3, 3), (1, 1), (1, 1), (1, 1)),     # 64x256, wgrad 64x192
    ((64, 64, 28, 28), (64, 64, 2, 2), (1, 1), (0, 0), (1, 1)),     # wgrad 64x128
    ((16, 128, 29, 29), (256, 128, 3, 3), (2, 2), (1, 1), (1, 1)),  # four dgrad phases, 128x64 tiles, tail slices
    ((4, 16, 15, 15), (32, 16, 3, 3), (1, 1), (1, 1), (1, 1)),      # 225 positions per sample (odd)
    ((6, 16, 20, 20), (10, 16, 3, 3), (1, 1), (1, 1), (1, 1)),      # F = 10: packed rows padded to 12
    ((5, 48, 9, 33), (16, 48, 3, 5), (1, 2), (1, 0), (1, 2)),       # 16-row tiles, dilation, mixed strides
    ((3, 32, 12, 12, 12), (32, 32, 3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),  # 3-D, 32-row tiles
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", range(len(KERNEL_VARIANT_CASES)))
def test_conv_shapes_that_reach_every_kernel_variant(abi, dtype, case):
    x_shape, w_shape, s, p, d = KERNEL_VARIANT_CASES[case]
    rng = np.random.default_rng(700 + case)
    tol = TOL[np.dtype(dtype)]
    print("variant case", np.dtype(dtype).name, x_shape, w_shape, s, p, d, flush=True)
    x = rng.standard_normal(x_shape).astype(dtype)
    w = (rng.standard_normal(w_shape) * (2.0 / np.prod(w_shape[1:])) ** 0.5).astype(dtype)
    want_out = direct.conv_forward(x, w, s, p, d)
    g = rng.standard_normal(want_out.shape).astype(dtype)
    assert rel_err(abi.conv_fwd(x, w, s, p, d), want_out) <= tol
    assert rel_err(abi.conv_dgrad(g, x_shape, w, s, p, d), direct.conv_backward_x(g, x_shape, w, s, p, d)) <= tol
    dw = abi.conv_wgrad(g, x, w_shape, s, p, d)
    assert rel_err(dw, direct.conv_backward_w(g, x, w_shape, s, p, d)) <= tol
    assert np.array_equal(bits(dw), bits(abi.conv_wgrad(g, x, w_shape, s, p, d)))  # fixed summation order


def _check_conv_config(abi, seed, dtype, x_shape, w_shape, w_scale, s, p, d, np_oracle_batch):
    """Full-size check: against the definition-level C reference everywhere, and
    against the NumPy restatement of the reference on the leading batch items."""
    rng = np.random.default_rng(seed)
    tol = TOL[np.dtype(dtype)]
    x = rng.standard_normal(x_shape).astype(dtype)
    w = (rng.standard_normal(w_shape) * w_scale).astype(dtype)
    out = abi.conv_fwd(x, w, s, p, d)
    g = rng.standard_normal(out.shape).astype(dtype)
    dx = abi.conv_dgrad(g, x_shape, w, s, p, d)
    dw = abi.conv_wgrad(g, x, w_shape, s, p, d)

    assert rel_err(out, direct.conv_forward(x, w, s, p, d)) <= tol
    assert rel_err(dx, direct.conv_backward_x(g, x_shape, w, s, p, d)) <= tol
    assert rel_err(dw, direct.conv_backward_w(g, x, w_shape, s, p, d)) <= tol

    # adjoint identity <conv(x,w), g> = <x, dx> = <w, dw>, in float64
    lhs = np.vdot(out.astype(np.float64), g.astype(np.float64))
    eps = 1e-9 if dtype == np.float64 else 1e-3
    scale = np.linalg.norm(out.astype(np.float64)) * np.linalg.norm(g.astype(np.float64))
    assert abs(lhs - np.vdot(x.astype(np.float64), dx.astype(np.float64))) <= eps * scale
    assert abs(lhs - np.vdot(w.astype(np.float64), dw.astype(np.float64))) <= eps * scale

    nb = np_oracle_batch
    conf = dict(stride=s, padding=p, dilation=d)
    ref_out = ora.conv_forward(x[:nb], w, validate=False, **conf)
    assert rel_err(out[:nb], ref_out) <= tol
    ref_dx = ora.conv_backward_x(g[:nb], x[:nb].shape, x.dtype, w, **conf)
    assert rel_err(dx[:nb], ref_dx) <= tol
    if nb == x_shape[0]:
        assert rel_err(dw, ora.conv_backward_w(g, x, w_shape, **conf)) <= tol


def test_conv_config1(abi):
    _check_conv_config(abi, 1001, np.float64, (32, 3, 32, 32), (16, 3, 3, 3), 1 / np.sqrt(27), (1, 1), (1, 1), (1, 1), 32)


def test_conv_config3a(abi):
    _check_conv_config(abi, 1003, np.float32, (128, 64, 56, 56), (64, 64, 3, 3), np.sqrt(2 / 576), (1, 1), (1, 1), (1, 1), 2)


def test_conv_config3b_literal(abi):
    _check_conv_config(abi, 1004, np.float32, (128, 128, 28, 28), (256, 128, 3, 3), np.sqrt(2 / 1152), (2, 2), (1, 1), (1, 1), 4)


def test_conv_config4_shape(abi):
    _check_conv_config(abi, 1005, np.float64, (16, 32, 128, 128), (32, 32, 5, 5), 1 / np.sqrt(800), (2, 1), (4, 4), (2, 2), 1)


def test_conv_config4_literal(abi):
    _check_conv_config(abi, 1005, np.float64, (16, 32, 128, 128), (32, 32, 5, 5), 1 / np.sqrt(800), (2, 1), (4, 2), (2, 2), 1)


def test_conv_config5(abi):
    _check_conv_config(abi, 1006, np.float32, (8, 16, 32, 64, 64), (32, 16, 3, 3, 3), np.sqrt(2 / 432), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1)


def test_conv_stem_three_channels_seven_by_seven_stride_two(abi):
    # a quarter of the batch of bench.py's `stem` workload, its literal (flooring) shape
    _check_conv_config(abi, 1017, np.float32, (32, 3, 224, 224), (64, 3, 7, 7), np.sqrt(2 / 147), (2, 2), (3, 3), (1, 1), 1)


def test_conv_wgrad_is_run_to_run_identical(abi):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((16, 24, 30, 30)).astype(np.float32)
    g = rng.standard_normal((16, 40, 28, 28)).astype(np.float32)
    first = abi.conv_wgrad(g, x, (40, 24, 3, 3), 1, 0, 1)
    for _ in range(3):
        assert np.array_equal(bits(first), bits(abi.conv_wgrad(g, x, (40, 24, 3, 3), 1, 0, 1)))


def test_abi_rejects_bad_arguments(abi):
    import ctypes

    from mygrad_amd import _hip

    lib = _hip.lib()
    desc, _ = abi.conv_desc((1, 1, 4, 4), (1, 1, 3, 3), np.float32, 1, 0, 1)
    assert lib.mg_conv_fwd(desc, None, None, None) == _hip.MG_ERR_BAD_ARG
    assert "null" in _hip.last_error()
    desc.dtype = 7
    assert lib.mg_conv_fwd(desc, 1, 1, 1) == _hip.MG_ERR_UNSUPPORTED
    desc.dtype = 0
    desc.G[2] = 99
    assert lib.mg_conv_fwd(desc, 1, 1, 1) == _hip.MG_ERR_BAD_ARG
    pdesc, _ = abi.pool_desc((2, 4, 4), np.float32, (2, 2), 2)
    pdesc.nd = 5
    assert lib.mg_maxpool_fwd(pdesc, 1, 1) == _hip.MG_ERR_UNSUPPORTED
    pdesc, _ = abi.pool_desc((2, 4, 4), np.float32, (2, 2), 2)
    assert lib.mg_maxpool_fwd_argmax(pdesc, 1, 1, None) == _hip.MG_ERR_BAD_ARG
    assert lib.mg_maxpool_bwd_argmax(pdesc, None, 1, 1) == _hip.MG_ERR_BAD_ARG
    wide, _ = abi.pool_desc((2, 20, 20), np.float32, (17, 16), 1)  # 272 positions: more than a byte tells apart
    assert lib.mg_maxpool_fwd_argmax(wide, 1, 1, 1) == _hip.MG_ERR_UNSUPPORTED
    assert lib.mg_maxpool_bwd_argmax(wide, 1, 1, 1) == _hip.MG_ERR_UNSUPPORTED
    assert "256" in _hip.last_error()
    huge = ctypes.c_void_p()
    assert lib.mg_malloc(ctypes.byref(huge), 1 << 60) == _hip.MG_ERR_OOM


def test_blocks_given_back_are_handed_out_again_in_stream_order(abi):
    """mg_free keeps the block, mg_malloc of a like size returns it without touching the
    driver; work enqueued on the block before it was given back runs before its next use."""
    import os

    from mygrad_amd import _device, _hip

    if os.environ.get("MYGRAD_HIP_POOL", "")[:1] == "0":
        pytest.skip("block reuse is switched off (MYGRAD_HIP_POOL=0)")
    size = 3 << 20
    first = _device.DeviceBuffer(size)
    ptr = first.ptr
    first.free()
    again = _device.DeviceBuffer(size - 4096)  # rounds to the same block size
    assert again.ptr == ptr
    # a kernel still writing the block when it is given back: the next owner's upload lands after it
    x = np.arange(size // 8, dtype=np.float64)
    src = _device.DeviceBuffer(size)
    src.upload(x)
    _hip.check(_hip.lib().mg_memcpy_d2d(again.ptr, src.ptr, size))  # enqueued, not waited for
    again.free()
    reused = _device.DeviceBuffer(size)
    assert reused.ptr == ptr
    reused.upload(-x)
    got = np.empty_like(x)
    reused.download_into(got)
    assert np.array_equal(got, -x)
    # a block of another size class does not take this one
    small = _device.DeviceBuffer(1024)
    assert small.ptr != ptr


@pytest.mark.gpu
def test_mfma_probe_reports_plausible_rates():
    """The diagnostic entry point runs and its figures are ordered the way the fp64
    kernels rely on: the four-block 4x4x4 MFMA outruns the 16x16x4 one."""
    from mygrad_amd import _hip

    f32 = _hip.probe_mfma("f32_16x16x4", 2)
    wide = _hip.probe_mfma("f64_16x16x4", 2)
    quad = _hip.probe_mfma("f64_4x4x4_4b", 2)
    assert 20.0 < f32 < 200.0 and 5.0 < wide < 100.0 and 5.0 < quad < 100.0
    assert quad > wide
    with pytest.raises(_hip.HipError):
        _hip.probe_mfma("f32_16x16x4", 9)


@pytest.mark.gpu
def test_stream_probe_moves_what_it_says():
    """The memory diagnostic stores every 16-byte piece of the large buffer from piece
    i / share of the small one (first value plus one), or loads the large buffer and stores
    every share-th piece to the small one; sizes and alignment are checked."""
    from mygrad_amd import _device, _hip

    pieces = 1000
    small_host = np.arange(4 * pieces, dtype=np.float32).reshape(pieces, 4)
    big, small = _device.DeviceBuffer(16 * pieces), _device.DeviceBuffer(16 * pieces)
    small.upload(small_host)
    got = np.empty((pieces, 4), dtype=np.float32)
    for share in (1, 2, 8):
        assert _hip.probe_stream(big.ptr, small.ptr, 16 * pieces, share, True) > 0.0
        big.download_into(got)
        want = small_host[np.arange(pieces) // share].copy()
        want[:, 0] += 1.0
        assert np.array_equal(got, want)
    _hip.probe_stream(big.ptr, small.ptr, 16 * pieces, 0, True)
    big.download_into(got)
    assert np.array_equal(got, np.tile(np.array([2.0, 2.0, 3.0, 4.0], dtype=np.float32), (pieces, 1)))
    big.upload(small_host)
    _hip.check(_hip.lib().mg_memset_zero(small.ptr, 16 * pieces))
    _hip.probe_stream(big.ptr, small.ptr, 16 * pieces, 4, False)
    small.download_into(got)
    assert np.array_equal(got[: pieces // 4], small_host[::4]) and not got[pieces // 4:].any()
    _hip.probe_stream(big.ptr, small.ptr, 16 * pieces, 0, False)  # loads only
    small.download_into(got)
    assert np.array_equal(got[: pieces // 4], small_host[::4])
    with pytest.raises(_hip.HipError):
        _hip.probe_stream(big.ptr, small.ptr, 24, 1, True)
    with pytest.raises(_hip.HipError):
        _hip.probe_stream(big.ptr + 4, small.ptr, 16, 1, True)


def test_per_launch_timing_records_chains_and_pauses():
    """``mg_timing_enable`` / ``mg_timing_read`` give one (kernel, milliseconds) record per timed
    launch, in order; ``mg_timing_pause`` suspends the recording without dropping what was
    recorded (what bench.py uses to time a sample of its steps)."""
    import mygrad_amd as mg
    from mygrad_amd import _hip

    a = mg.device_tensor(np.ones((256, 1024), dtype=np.float32))
    b = mg.device_tensor(np.full((256, 1024), 2.0, dtype=np.float32))
    with mg.no_autodiff:
        _hip.timing_enable(True)
        try:
            mg.multiply(a, b)
            _hip.timing_pause(True)
            for _ in range(3):
                mg.multiply(a, b)
            _hip.timing_pause(False)
            mg.multiply(a, b)
            mg.multiply(a, b)
            records = _hip.timing_read()
        finally:
            _hip.timing_enable(False)
    assert [k for k, _ in records] == ["elementwise"] * 3
    assert all(0.0 < ms < 5.0 for _, ms in records)
    with mg.no_autodiff:
        mg.multiply(a, b)  # timing off: nothing is recorded, nothing is left over
    _hip.timing_enable(True)
    try:
        assert _hip.timing_read() == []
    finally:
        _hip.timing_enable(False)
