"""Parity of batch normalisation (forward, and the gradients in x, gamma and beta) with the
NumPy restatement of the reference, through the C ABI and through ``Tensor.backward()``.

Bars (maximum absolute error over the array, relative to the largest magnitude of the
expected array): 1e-10 in float64; in float32 1e-5 against the float64 result for the
statistics and 2e-5 for the normalised batch and the gradients.  Results are identical
from run to run (fixed partition, fixed trees, no atomics)."""

import numpy as np
import pytest

from oracle import np_oracle as ora

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 2e-5, np.dtype(np.float64): 1e-10}
STAT_TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}


@pytest.fixture(scope="module")
def abi():
    import mygrad_amd

    if not mygrad_amd.is_available():
        pytest.fail("libmygrad_hip.so / gfx950 device not available: the GPU tests need both")
    from tests import abi as module

    return module


def err(got, want):
    want = np.asarray(want, dtype=np.float64)
    scale = float(np.max(np.abs(want))) or 1.0
    return float(np.max(np.abs(np.asarray(got, dtype=np.float64) - want))) / scale


# shapes: no trailing axes and short rows (walked by columns, one or many pieces of the batch
# axis), rows that are / are not a whole number of 16-byte pieces, fewer elements per channel
# than one block, many chunks per channel, one channel, many
SHAPES = [
    (3, 1),
    (5, 3),
    (4096, 512),
    (70000, 2),
    (300, 7, 5),
    (2, 3, 33),
    (1, 4, 7),
    (4, 3, 8),
    (2, 5, 3, 5),
    (8, 16, 12, 12),
    (2, 3, 4, 6, 6),
    (64, 1, 56, 56),
    (2, 1000, 3, 3),
    (16, 8, 55, 55),
    (8, 4, 128, 128),
]


def _case(shape, dtype, seed):
    rng = np.random.default_rng([seed, len(shape), int(np.prod(shape))])
    channels = shape[1]
    keep = (1, channels) + (1,) * (len(shape) - 2)
    x = rng.standard_normal(shape) * rng.uniform(0.5, 3, channels).reshape(keep) + rng.uniform(-3, 3, channels).reshape(keep)
    gamma = rng.uniform(0.5, 2, channels) * rng.choice([-1.0, 1.0], channels)
    beta = rng.uniform(-2, 2, channels)
    grad = rng.standard_normal(shape)
    return x.astype(dtype), gamma.astype(dtype), beta.astype(dtype), grad.astype(dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("affine", [(False, False), (True, True), (True, False), (False, True)])
def test_forward_and_backward_match_the_oracle(abi, shape, dtype, affine):
    dtype = np.dtype(dtype)
    x, gamma, beta, grad = _case(shape, dtype, 1)
    gamma = gamma if affine[0] else None
    beta = beta if affine[1] else None
    eps = 1e-5
    y, mean, var = abi.batchnorm_fwd(x, gamma, beta, eps=eps)
    wide = [None if a is None else a.astype(np.float64) for a in (x, gamma, beta, grad)]
    want_y, want_mean, want_var = ora.batchnorm_forward(wide[0], wide[1], wide[2], eps=eps)
    assert y.dtype == mean.dtype == var.dtype == dtype
    assert err(mean, want_mean) <= STAT_TOL[dtype] and err(var, want_var) <= STAT_TOL[dtype]
    assert err(y, want_y) <= TOL[dtype]
    if dtype == np.float32:  # and the reference's own float32 arithmetic agrees to the same bar
        same_y, same_mean, same_var = ora.batchnorm_forward(x, gamma, beta, eps=eps)
        assert same_y.dtype == np.float32
        assert err(y, same_y) <= TOL[dtype] and err(mean, same_mean) <= 1e-4 and err(var, same_var) <= 1e-4

    dx, dgamma, dbeta = abi.batchnorm_bwd(grad, x, mean, var, gamma, eps=eps)
    want_dx, want_dgamma, want_dbeta = ora.batchnorm_backward(wide[3], wide[0], wide[1], eps=eps)
    assert err(dx, want_dx) <= TOL[dtype]
    # channel sums are compared against the size of what was summed
    xn = ora.batchnorm_forward(wide[0], eps=eps)[0]
    axes = tuple(i for i in range(x.ndim) if i != 1)
    assert np.all(np.abs(dgamma - want_dgamma) <= TOL[dtype] * np.maximum(np.abs(wide[3] * xn).sum(axis=axes), 1e-30))
    assert np.all(np.abs(dbeta - want_dbeta) <= TOL[dtype] * np.maximum(np.abs(wide[3]).sum(axis=axes), 1e-30))


def test_reference_docstring_vector(abi, kats):
    for case in kats["batchnorm"]:
        for dtype in (np.float32, np.float64):
            y, mean, var = abi.batchnorm_fwd(np.array(case["x"], dtype=dtype), eps=case["eps"])
            assert np.allclose(y, np.array(case["out"]), rtol=0, atol=2e-8 if dtype == np.float64 else 1e-6)
            assert mean[0] == 2.0 and var[0] == 2.0


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_statistics_survive_a_large_offset(abi, dtype):
    """|mean| / std = 1e3 (float32) or 1e7 (float64): sums of squares about zero would lose
    the variance; sums about a pilot value near the mean do not."""
    dtype = np.dtype(dtype)
    rng = np.random.default_rng(5)
    offset = 1e3 if dtype == np.float32 else 1e7
    x = (rng.standard_normal((16, 3, 40, 40)) + offset).astype(dtype)
    _, mean, var = abi.batchnorm_fwd(x, eps=0.0)
    wide = x.astype(np.float64)
    want_mean = wide.mean(axis=(0, 2, 3))
    want_var = ((wide - want_mean.reshape(1, 3, 1, 1)) ** 2).mean(axis=(0, 2, 3))
    assert err(mean, want_mean) <= (1e-7 if dtype == np.float32 else 1e-15)
    assert err(var, want_var) <= (1e-6 if dtype == np.float32 else 1e-12)


def test_constant_channel_and_single_element_channels(abi):
    x = np.full((4, 2, 5), 3.25)
    x[:, 1] = np.arange(20.0).reshape(4, 5)
    y, mean, var = abi.batchnorm_fwd(x, eps=1e-3)
    assert np.array_equal(y[:, 0], np.zeros((4, 5))) and mean[0] == 3.25 and var[0] == 0.0
    want = ora.batchnorm_forward(x, eps=1e-3)
    assert err(y, want[0]) <= 1e-12 and err(var, want[2]) <= 1e-12
    one = np.array([[1.5, -2.0, 7.0]])  # one element per channel: y = 0 / sqrt(eps)
    y, mean, var = abi.batchnorm_fwd(one, eps=0.25)
    assert np.array_equal(y, np.zeros((1, 3))) and np.array_equal(mean, one[0]) and np.array_equal(var, np.zeros(3))
    with np.errstate(invalid="ignore"):
        y, _, _ = abi.batchnorm_fwd(one, eps=0.0)  # 0 / 0, as in the reference
    assert np.isnan(y).all()


@pytest.mark.parametrize("bad", [np.nan, np.inf])
@pytest.mark.parametrize("shape, where", [((6, 3, 20, 20), (4, 1, 7, 3)), ((500, 3), (321, 1))])
def test_a_non_finite_element_poisons_its_own_channel_only(abi, bad, shape, where):
    """As in the reference: the channel's mean, variance and normalised values become NaN
    (an infinite mean for an infinite element), the other channels are untouched."""
    x, _, _, _ = _case(shape, np.dtype(np.float64), 9)
    clean = abi.batchnorm_fwd(x, eps=1e-5)
    x[where] = bad
    with np.errstate(invalid="ignore"):
        y, mean, var = abi.batchnorm_fwd(x, eps=1e-5)
        want_y, want_mean, want_var = ora.batchnorm_forward(x, eps=1e-5)
    assert np.isnan(want_var[1]) and np.isnan(var[1]) and np.isnan(y[:, 1]).all()
    assert np.isnan(mean[1]) if np.isnan(want_mean[1]) else mean[1] == want_mean[1]
    for c in (0, 2):
        assert np.array_equal(y[:, c], clean[0][:, c]) and mean[c] == clean[1][c] and var[c] == clean[2][c]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_results_are_identical_from_run_to_run_and_outputs_are_optional(abi, dtype):
    x, gamma, beta, grad = _case((8, 6, 30, 30), np.dtype(dtype), 3)
    first = abi.batchnorm_fwd(x, gamma, beta, eps=1e-5)
    again = abi.batchnorm_fwd(x, gamma, beta, eps=1e-5)
    assert all(np.array_equal(a, b) for a, b in zip(first, again))
    _, mean, var = first
    full = abi.batchnorm_bwd(grad, x, mean, var, gamma, eps=1e-5)
    for want in (("x",), ("gamma",), ("beta",), ("gamma", "beta"), ("x", "beta"), ("x", "gamma", "beta")):
        part = abi.batchnorm_bwd(grad, x, mean, var, gamma, eps=1e-5, want=want)
        for name, got, ref in zip(("x", "gamma", "beta"), part, full):
            assert (got is None) == (name not in want)
            assert got is None or np.array_equal(got, ref)


def test_abi_rejects_bad_arguments(abi):
    from mygrad_amd import _device, _hip

    buf = _device.DeviceBuffer(4096)
    lib = _hip.lib()
    p = buf.ptr
    good = _hip.bn_desc((2, 3, 4), np.float32, False, False, 1e-5)
    assert lib.mg_batchnorm_fwd(good, p, None, None, p, p, p) == 0
    assert lib.mg_batchnorm_fwd(None, p, None, None, p, p, p) == -1
    assert lib.mg_batchnorm_fwd(good, None, None, None, p, p, p) == -1
    assert lib.mg_batchnorm_fwd(_hip.bn_desc((2, 3, 4), np.float32, True, False, 1e-5), p, None, None, p, p, p) == -1
    assert lib.mg_batchnorm_fwd(_hip.bn_desc((2, 3, 4), np.float32, False, False, -1.0), p, None, None, p, p, p) == -1
    assert lib.mg_batchnorm_fwd(_hip.bn_desc((2, 0, 4), np.float32, False, False, 0.0), p, None, None, p, p, p) == -1
    bad = _hip.bn_desc((2, 3, 4), np.float32, False, False, 1e-5)
    bad.dtype = 7
    assert lib.mg_batchnorm_fwd(bad, p, None, None, p, p, p) == -2
    assert lib.mg_batchnorm_bwd(good, p, p, None, p, p, None, None, None) == -1
    assert b"nothing to compute" in lib.mg_last_error()


# ------------------------------------------------------------------ through the drop-in
def test_batchnorm_through_the_tensor_api():
    import mygrad_amd as mg
    from mygrad_amd import _graph
    from mygrad_amd.nnet import batchnorm

    y = batchnorm(mg.Tensor([[1.0], [4.0], [1.0]]), eps=0)
    assert np.allclose(y.data, [[-0.70710678], [1.41421356], [-0.70710678]], atol=2e-8)
    assert y.creator.mean.shape == (1,) and y.creator.mean[0] == 2.0 and y.creator.var[0] == 2.0
    y.backward()  # releases the graph (and the read-only hold on its arrays)

    for dtype in (np.float64, np.float32):
        xd, gd, bd, grad = _case((4, 5, 6, 7), np.dtype(dtype), 9)
        x, gamma, beta = mg.Tensor(xd), mg.Tensor(gd), mg.Tensor(bd)
        out = batchnorm(x, gamma=gamma, beta=beta, eps=1e-6)
        want = ora.batchnorm_forward(xd.astype(np.float64), gd.astype(np.float64), bd.astype(np.float64), eps=1e-6)
        assert out.dtype == dtype and err(out.data, want[0]) <= TOL[np.dtype(dtype)]
        out.backward(grad)
        dx, dgamma, dbeta = ora.batchnorm_backward(grad.astype(np.float64), xd.astype(np.float64), gd.astype(np.float64), eps=1e-6)
        assert x.grad.dtype == gamma.grad.dtype == beta.grad.dtype == dtype
        assert err(x.grad, dx) <= TOL[np.dtype(dtype)]
        assert err(gamma.grad, dgamma) <= 10 * TOL[np.dtype(dtype)] and err(beta.grad, dbeta) <= 10 * TOL[np.dtype(dtype)]
        assert not np.shares_memory(gamma.grad, beta.grad)
        assert not x._ops and not gamma._ops and not beta._ops

        # beta alone is the second variable's slot holder when there is no gamma (batchnorm.py:104)
        x, beta = mg.Tensor(xd), mg.Tensor(bd)
        out = batchnorm(x, beta=beta, eps=1e-6)
        out.backward(grad)
        dx, _, dbeta = ora.batchnorm_backward(grad.astype(np.float64), xd.astype(np.float64), eps=1e-6)
        assert err(x.grad, dx) <= TOL[np.dtype(dtype)] and err(beta.grad, dbeta) <= 10 * TOL[np.dtype(dtype)]

        # a constant x still gives gamma its gradient
        gamma = mg.Tensor(gd)
        out = batchnorm(mg.Tensor(xd, constant=True), gamma=gamma, eps=1e-6)
        out.backward(grad)
        assert err(gamma.grad, dgamma) <= 10 * TOL[np.dtype(dtype)]
    assert _graph.held_count() == 0

    assert batchnorm(mg.Tensor(xd), eps=1e-6, constant=True).constant
    with pytest.raises(TypeError):
        batchnorm(mg.Tensor(xd.astype(np.float32)), gamma=gd.astype(np.float64), eps=1e-6)
    with pytest.raises(ValueError):
        batchnorm(mg.Tensor(xd), gamma=gd[:-1], eps=1e-6)
    with pytest.raises(ValueError):
        batchnorm(mg.Tensor(np.ones(4)), eps=1e-6)
    with pytest.raises(TypeError):
        batchnorm(mg.Tensor(np.ones((4, 2), dtype=np.int64)), eps=1e-6)


def test_conv_batchnorm_relu_pool_chain_stays_on_the_device():
    """conv -> batchnorm -> relu -> max_pool, the ResNet-style block: intermediate results
    are handed from kernel to kernel in device memory (uploads: x, w, gamma, beta, seed)."""
    import mygrad_amd as mg
    from mygrad_amd import _device
    from mygrad_amd.nnet import batchnorm, conv_nd, max_pool, relu

    rng = np.random.default_rng(12)
    x = mg.Tensor(rng.standard_normal((4, 8, 16, 16)))
    w = mg.Tensor(rng.standard_normal((16, 8, 3, 3)) * (2 / 72) ** 0.5)
    gamma, beta = mg.Tensor(rng.uniform(0.5, 2, 16)), mg.Tensor(rng.standard_normal(16))
    seed = rng.standard_normal((4, 16, 8, 8))
    before = dict(_device.stats)
    y = conv_nd(x, w, stride=1, padding=1)
    b = batchnorm(y, gamma=gamma, beta=beta, eps=1e-5)
    z = max_pool(relu(b), (2, 2), 2)
    y_data, b_data = y.data, b.data
    z.backward(seed)
    assert _device.stats["uploads"] - before["uploads"] == 5

    want_b = ora.batchnorm_forward(y_data, gamma.data, beta.data, eps=1e-5)[0]
    assert err(b_data, want_b) <= 1e-10
    want_db = ora.relu_backward(b_data, ora.pool_backward(ora.relu_forward(b_data), seed, (2, 2), 2))
    want_dy, want_dgamma, want_dbeta = ora.batchnorm_backward(want_db, y_data, gamma.data, eps=1e-5)
    assert err(y.grad, want_dy) <= 1e-10
    assert err(gamma.grad, want_dgamma) <= 1e-10 and err(beta.grad, want_dbeta) <= 1e-10
    want_dx = ora.conv_backward_x(want_dy, x.shape, x.dtype, w.data, stride=1, padding=1)
    want_dw = ora.conv_backward_w(want_dy, x.data, w.shape, stride=1, padding=1)
    assert err(x.grad, want_dx) <= 1e-10 and err(w.grad, want_dw) <= 1e-10
