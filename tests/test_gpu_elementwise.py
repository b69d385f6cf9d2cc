"""Parity of the element-wise and whole-array kernels (multiply, relu, sum) that sit either
side of conv_nd / max_pool, through the C ABI and through ``Tensor.backward()``.

Bars: multiply and relu bit-exact (one IEEE operation per element, special values
included); sum within 1e-6 (float32) / 1e-14 (float64) of the exact sum relative to
sum|x|, and identical from run to run."""

import math

import numpy as np
import pytest

from oracle import direct
from oracle import np_oracle as ora

pytestmark = pytest.mark.gpu

SUM_TOL = {np.dtype(np.float32): 1e-6, np.dtype(np.float64): 1e-14}


@pytest.fixture(scope="module")
def abi():
    import mygrad_amd

    if not mygrad_amd.is_available():
        pytest.fail("libmygrad_hip.so / gfx950 device not available: the GPU tests need both")
    from tests import abi as module

    return module


def bits(a):
    return a.view(np.uint32 if a.dtype == np.float32 else np.uint64)


def _specials(rng, shape, dtype):
    x = rng.standard_normal(shape).astype(dtype)
    flat = x.reshape(-1)
    for value in (np.nan, np.inf, -np.inf, 0.0, -0.0, np.finfo(dtype).tiny / 4, np.finfo(dtype).max):
        flat[rng.integers(0, flat.size, max(1, flat.size // 50))] = value
    return x


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape", [(1,), (3,), (257,), (5, 7, 11), (2, 3, 64, 65), (1 << 20,)])
def test_multiply_and_relu_bit_exact(abi, dtype, shape):
    rng = np.random.default_rng(900 + len(shape) + shape[-1] % 97)
    a, b, g = (_specials(rng, shape, dtype) for _ in range(3))
    with np.errstate(all="ignore"):
        assert np.array_equal(bits(abi.multiply(a, b)), bits(ora.multiply(a, b)))
        assert np.array_equal(bits(abi.relu_fwd(a)), bits(ora.relu_forward(a)))
        assert np.array_equal(bits(abi.relu_bwd(a, g)), bits(ora.relu_backward(a, g)))


def test_relu_reference_docstring_vectors(abi, kats):
    for case in kats["relu"]:
        x = np.array(case["x"])
        out = abi.relu_fwd(x)
        assert np.array_equal(out, np.array(case["out"])) and np.array_equal(np.signbit(out), case["out_signbit"])
        assert np.array_equal(abi.relu_bwd(x, np.ones_like(x)), np.array(case["dx_of_ones"]))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [1, 2, 5, 4096, 16384 + 3, 1 << 20, (1 << 24) + 7, 80_000_001])
def test_sum_against_the_exact_sum(abi, dtype, n):
    rng = np.random.default_rng(n % 1000)
    x = (rng.standard_normal(n) * 10.0 ** rng.integers(-3, 4, n)).astype(dtype)
    got = abi.sum_all(x)
    assert got.dtype == dtype and got.shape == ()
    exact = math.fsum(x.astype(np.float64)) if n <= (1 << 20) else float(np.sum(x.astype(np.longdouble)))
    scale = float(np.sum(np.abs(x.astype(np.float64))))
    assert abs(float(got) - exact) <= SUM_TOL[np.dtype(dtype)] * scale
    assert abs(float(got) - float(ora.sum_all(x))) <= 2 * SUM_TOL[np.dtype(dtype)] * scale
    assert bits(np.asarray(abi.sum_all(x)).reshape(1))[0] == bits(np.asarray(got).reshape(1))[0]  # same tree every run


def test_sum_closed_forms_and_fill(abi):
    n = 100001
    assert float(abi.sum_all(np.arange(n, dtype=np.float64))) == n * (n - 1) / 2
    assert float(abi.sum_all(np.ones(12345, dtype=np.float32))) == 12345.0
    for dtype in (np.float32, np.float64):
        for shape in ((1,), (7,), (3, 5, 9), (2, 1 << 18)):
            want = ora.sum_all_backward(np.empty(shape, dtype), 2.5)
            assert np.array_equal(abi.fill_from(2.5, shape, dtype), want)


def test_abi_rejects_bad_arguments(abi):
    from mygrad_amd import _device, _hip

    buf = _device.DeviceBuffer(64)
    lib = _hip.lib()
    assert lib.mg_multiply(5, 4, buf.ptr, buf.ptr, buf.ptr) == -2
    assert lib.mg_multiply(0, -1, buf.ptr, buf.ptr, buf.ptr) == -1
    assert lib.mg_relu_fwd(0, 4, None, buf.ptr) == -1
    assert lib.mg_sum_all(1, 4, buf.ptr + 8, buf.ptr) == -1  # misaligned
    assert lib.mg_sum_all(1, 0, None, buf.ptr) == 0
    assert lib.mg_fill_from(0, 4, None, buf.ptr) == -1


# ------------------------------------------------------------------ through the drop-in
def test_docstring_examples_through_the_tensor_api():
    import mygrad_amd as mg
    from mygrad_amd.nnet import relu

    x = mg.Tensor([-5.0, -2.5, 0.0, 2.5, 5.0])
    y = relu(x)
    assert np.array_equal(y.data, [-0.0, -0.0, 0.0, 2.5, 5.0]) and np.signbit(y.data[:2]).all()
    y.backward()
    assert np.array_equal(x.grad, [0.0, 0.0, 0.0, 1.0, 1.0])

    a, b = mg.Tensor([1.0, 2.0, 3.0]), mg.Tensor([4.0, 5.0, 6.0])
    s = mg.sum(a * b)
    assert s.data.shape == () and float(s.data) == 32.0
    s.backward()
    assert np.array_equal(a.grad, [4.0, 5.0, 6.0]) and np.array_equal(b.grad, [1.0, 2.0, 3.0])

    with pytest.raises(NotImplementedError):
        mg.multiply(mg.Tensor(np.ones((2, 3))), np.ones(3))
    with pytest.raises(NotImplementedError):
        mg.sum(mg.Tensor(np.ones((2, 3))), axis=0)
    with pytest.raises(TypeError):
        relu(mg.Tensor(np.arange(4)))


def test_conv_relu_pool_multiply_sum_chain_stays_on_the_device():
    """loss = sum(max_pool(relu(conv_nd(x, w))) * g): the chain of the 3-D benchmark
    configuration with the loss formed on the device; only x, w and g are uploaded."""
    import mygrad_amd as mg
    from mygrad_amd import _device, _graph
    from mygrad_amd.nnet import conv_nd, max_pool, relu

    rng = np.random.default_rng(1006)
    dtype = np.float32
    x = mg.Tensor(rng.standard_normal((2, 16, 8, 32, 32)).astype(dtype))
    w = mg.Tensor((rng.standard_normal((32, 16, 3, 3, 3)) * (2 / 432) ** 0.5).astype(dtype))
    g = mg.Tensor(rng.standard_normal((2, 32, 4, 16, 16)).astype(dtype), constant=True)
    before = dict(_device.stats)
    y = conv_nd(x, w, stride=1, padding=1)
    r = relu(y)
    z = max_pool(r, (2, 2, 2), 2)
    loss = mg.sum(z * g)
    y_data, r_data, z_data, loss_value = y.data, r.data, z.data, float(loss.data)
    loss.backward()
    assert _device.stats["uploads"] - before["uploads"] == 4  # x, w, g and the seed gradient 1.0

    s = p = d = (1, 1, 1)
    want_y = direct.conv_forward(x.data, w.data, s, p, d)
    assert float(np.max(np.abs(y_data - want_y))) <= 2e-4 * float(np.max(np.abs(want_y)))
    assert np.array_equal(bits(r_data), bits(ora.relu_forward(y_data)))
    want_z, _ = direct.pool(r_data, g.data, (2, 2, 2), (2, 2, 2))
    assert np.array_equal(z_data, want_z)
    prod = z_data.astype(np.float64) * g.data.astype(np.float64)
    assert abs(loss_value - float(prod.sum())) <= 1e-6 * float(np.abs(prod).sum())
    # backward: d loss / d z = g exactly, routed by the pool, masked by relu, then the conv gradients
    _, want_dr = direct.pool(r_data, g.data, (2, 2, 2), (2, 2, 2))
    want_dy = ora.relu_backward(y_data, want_dr.astype(dtype))
    assert np.array_equal(bits(y.grad), bits(want_dy))
    want_dx = direct.conv_backward_x(want_dy, x.shape, w.data, s, p, d)
    want_dw = direct.conv_backward_w(want_dy, x.data, w.shape, s, p, d)
    assert float(np.max(np.abs(x.grad - want_dx))) <= 2e-4 * float(np.max(np.abs(want_dx)))
    assert float(np.max(np.abs(w.grad - want_dw))) <= 2e-4 * float(np.max(np.abs(want_dw)))
    assert _graph.held_count() == 0
