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
        # the pair that keeps the mask (one bit per element) between the passes
        out, mask = abi.relu_fwd_mask(a)
        assert np.array_equal(bits(out), bits(ora.relu_forward(a)))
        assert np.array_equal(mask, np.packbits(a.reshape(-1) > 0, bitorder="little"))
        assert np.array_equal(bits(abi.relu_bwd_mask(mask, g)), bits(ora.relu_backward(a, g)))


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


SUM_OVER_SHAPES = [
    (1, 1, 1), (3, 1, 5), (1, 7, 1), (5, 3, 1), (1, 4, 9), (6, 5, 4), (2, 3, 64), (128, 64, 3136 // 16),
    (70000, 3, 1), (1, 70000, 3), (4, 70000, 64), (3, 2, 100003), (40000, 5, 2), (2, 100000, 4), (1, 1000, 1000),
    (500, 33, 130), (9, 4000, 7),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape", SUM_OVER_SHAPES)
def test_sum_over_both_forms_against_exact_sums(abi, dtype, shape):
    """mg_sum_over: x:(outer, n, inner) summed over the middle axis, and over the two outer
    ones.  Bar: |got - exact| <= 1e-6 (float32) / 1e-14 (float64) of the sum of magnitudes
    of what was added, the exact sum being NumPy's in extended precision; and the same
    against np.sum in the array's own precision, with twice the allowance."""
    dtype = np.dtype(dtype)
    rng = np.random.default_rng(list(shape))
    x = (rng.standard_normal(shape) * 10.0 ** rng.integers(-2, 3, shape)).astype(dtype)
    wide = x.astype(np.longdouble)
    for over_middle, axes in ((True, (1,)), (False, (0, 2))):
        got = abi.sum_over(x, over_middle)
        exact = wide.sum(axis=axes)
        scale = np.abs(wide).sum(axis=axes) + 1e-300
        assert got.dtype == dtype and got.shape == exact.shape
        assert np.all(np.abs(got - exact) <= SUM_TOL[dtype] * scale)
        assert np.all(np.abs(got - ora.sum_axes(x, axes)) <= 2 * SUM_TOL[dtype] * scale)
        assert np.array_equal(bits(abi.sum_over(x, over_middle)), bits(got))  # the same partition and trees every run


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape", SUM_OVER_SHAPES)
def test_sum_product_over_equals_product_then_sum(abi, dtype, shape):
    """mg_sum_product_over rounds each product to the array's precision before adding it and
    adds in mg_sum_over's order, so it gives bit for bit what mg_multiply followed by
    mg_sum_over gives (both of which are checked against NumPy on their own)."""
    dtype = np.dtype(dtype)
    rng = np.random.default_rng([3, *shape])
    x = (rng.standard_normal(shape) * 10.0 ** rng.integers(-2, 3, shape)).astype(dtype)
    y = rng.standard_normal(shape).astype(dtype)
    product = abi.multiply(x, y)
    assert np.array_equal(bits(product), bits(x * y))
    for over_middle in (True, False):
        got = abi.sum_product_over(x, y, over_middle)
        assert np.array_equal(bits(got), bits(abi.sum_over(product, over_middle)))


def test_sum_product_over_bad_arguments(abi):
    from mygrad_amd import _device, _hip

    buf, lib = _device.DeviceBuffer(64), _hip.lib()
    assert lib.mg_sum_product_over(0, 1, 2, 3, 0, buf.ptr, None, buf.ptr) == _hip.MG_ERR_BAD_ARG
    assert lib.mg_sum_product_over(0, 1, 2, 3, 0, None, buf.ptr, buf.ptr) == _hip.MG_ERR_BAD_ARG
    assert lib.mg_sum_product_over(0, 1, 0, 3, 1, buf.ptr, buf.ptr, buf.ptr) == _hip.MG_ERR_BAD_ARG
    assert lib.mg_sum_product_over(2, 1, 2, 3, 1, buf.ptr, buf.ptr, buf.ptr) == _hip.MG_ERR_UNSUPPORTED
    assert "mg_sum_product_over" in _hip.last_error()


def test_sum_over_full_size(abi):
    """The benchmark's tensor (134 MB) summed per channel and over the channel axis, against
    NumPy's sums of the same values in float64."""
    rng = np.random.default_rng(94)
    x = rng.standard_normal((8, 32, 32 * 64 * 64), dtype=np.float32)
    wide = x.astype(np.float64)
    for over_middle, axes in ((False, (0, 2)), (True, (1,))):
        got = abi.sum_over(x, over_middle)
        want = wide.sum(axis=axes)
        scale = np.abs(wide).sum(axis=axes)
        assert np.all(np.abs(got - want) <= SUM_TOL[np.dtype(np.float32)] * scale)


def test_sum_over_closed_forms_and_bad_arguments(abi):
    from mygrad_amd import _device, _hip

    x = np.arange(2 * 3 * 4, dtype=np.float64).reshape(2, 3, 4)
    assert np.array_equal(abi.sum_over(x, True), x.sum(axis=1))
    assert np.array_equal(abi.sum_over(x, False), x.sum(axis=(0, 2)))
    ones = np.ones((300, 70, 50), dtype=np.float32)
    assert np.array_equal(abi.sum_over(ones, True), np.full((300, 50), 70.0, np.float32))
    assert np.array_equal(abi.sum_over(ones, False), np.full(70, 15000.0, np.float32))
    nan = np.ones((4, 3, 5))
    nan[2, 1, 3] = np.nan
    assert np.isnan(abi.sum_over(nan, False)[1]) and np.isnan(abi.sum_over(nan, True)[2, 3])
    assert np.isnan(abi.sum_over(nan, True)).sum() == 1 and np.isnan(abi.sum_over(nan, False)).sum() == 1
    buf = _device.DeviceBuffer(64)
    lib = _hip.lib()
    assert lib.mg_sum_over(0, 1, 2, 3, 0, None, buf.ptr) == _hip.MG_ERR_BAD_ARG
    assert lib.mg_sum_over(0, 0, 2, 3, 1, buf.ptr, buf.ptr) == _hip.MG_ERR_BAD_ARG
    assert lib.mg_sum_over(3, 1, 2, 3, 1, buf.ptr, buf.ptr) == _hip.MG_ERR_UNSUPPORTED


TENSOR_SUM_CASES = [
    ((4, 5), 0, False), ((4, 5), -1, True), ((2, 3, 4), (0, 2), False), ((2, 3, 4), (1,), True), ((2, 1, 3, 2), (1, 3), False),
    ((3,), None, True), ((2, 3, 2, 2, 3), (1, 3), True), ((2, 3), (), False), ((2, 3, 4, 5, 2), (0, 2, 4), False),
    ((8, 16, 12, 12), (0, 2, 3), False), ((8, 16, 12, 12), 1, True), ((64, 1000), 0, False), ((64, 1000), 1, False),
    ((1, 5, 1), (0, 2), False), ((0, 3), 0, False), ((0, 3), 1, True), ((), None, False),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape,axis,keepdims", TENSOR_SUM_CASES)
def test_sum_over_axes_through_the_tensor_api(dtype, shape, axis, keepdims):
    import mygrad_amd as mg

    dtype = np.dtype(dtype)
    rng = np.random.default_rng([len(shape), int(np.prod(shape)), 5])
    xv = rng.standard_normal(shape).astype(dtype)
    x = mg.Tensor(xv)
    out = mg.sum(x, axis=axis, keepdims=keepdims)
    want = ora.sum_axes(xv, axis, keepdims)
    assert out.shape == want.shape and out.dtype == want.dtype
    scale = np.abs(xv.astype(np.float64)).sum(axis=axis, keepdims=keepdims)
    assert np.all(np.abs(out.data.astype(np.float64) - want) <= 2 * SUM_TOL[dtype] * (scale + 1e-300))
    g = rng.standard_normal(want.shape).astype(dtype)
    out.backward(g)
    back = ora.sum_axes_backward(xv, g, axis, keepdims)
    assert x.grad.dtype == back.dtype and np.array_equal(x.grad, back)  # a copy of values: exact


def test_sum_axis_errors_through_the_tensor_api():
    import mygrad_amd as mg

    x = mg.Tensor(np.ones((2, 3)))
    with pytest.raises(np.exceptions.AxisError):
        mg.sum(x, axis=2)
    with pytest.raises(ValueError):
        mg.sum(x, axis=(0, 0))
    assert float(mg.sum(mg.Tensor(3.0), axis=0).data) == 3.0


BROADCAST_CASES = [
    ((4, 5), (5,)), ((4, 5), (4, 1)), ((2, 3, 4), (3, 1)), ((3, 1, 2), (1, 4, 1)), ((2, 3), ()), ((1,), (2, 3)),
    ((2, 3, 4, 5), (1, 3, 1, 1)), ((5,), (5,)), ((8, 16, 12, 12), (16, 1, 1)), ((64, 1000), (1000,)), ((64, 1000), (64, 1)),
    ((2, 1, 3, 1, 2), (3, 1, 4, 1)), ((0, 3), (3,)), ((2, 3), (1,)),
    # rows of whole 16-byte pieces with either operand, or neither, along them; rows that are not
    ((6, 1, 64), (1, 5, 64)), ((6, 5, 1), (1, 1, 64)), ((3, 7, 1), (7, 62)), ((16, 1), (1, 16)), ((1, 1), (1,)),
    ((4, 1, 6, 1, 8), (3, 1, 5, 1)), ((2, 1, 2, 1, 2, 1), (1, 3, 1, 3, 1, 8)),
    # seven groups of axes after merging: more than the one-pass kernel takes, the operands are spread first
    ((2, 1, 2, 1, 2, 1, 2), (1, 3, 1, 3, 1, 3, 1)),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("sa,sb", [c for c in BROADCAST_CASES if 0 not in c[0] + c[1]])
def test_multiply_broadcast_bit_exact(abi, dtype, sa, sb):
    rng = np.random.default_rng([7, len(sa), len(sb), int(np.prod(sa)) + int(np.prod(sb))])
    a, b = rng.standard_normal(sa).astype(dtype), rng.standard_normal(sb).astype(dtype)
    flat = a.reshape(-1)  # a view: special values at both ends and in the middle
    flat[0], flat[-1], flat[a.size // 2] = np.nan, -0.0, np.inf
    got = abi.multiply_broadcast(a, b)
    from mygrad_amd import _reduce

    if len(_reduce.multiply_plan(sa, sb, np.broadcast_shapes(sa, sb))[0]) > _reduce.MAX_MULTIPLY_AXES:
        assert got is None
        return
    with np.errstate(invalid="ignore"):
        want = ora.multiply(a, b)
    assert got.shape == want.shape and np.array_equal(bits(got), bits(want))


def test_multiply_broadcast_rejects_bad_arguments(abi):
    import ctypes

    from mygrad_amd import _device, _hip

    lib, buf = _hip.lib(), _device.DeviceBuffer(4096)
    arr = lambda *v: (ctypes.c_int64 * len(v))(*v)
    call = lambda nd, shape, sa, sb, dtype=0: lib.mg_multiply_broadcast(dtype, nd, shape, sa, sb, buf.ptr, buf.ptr, buf.ptr)
    assert call(2, arr(4, 8), arr(8, 1), arr(0, 1)) == _hip.MG_OK
    assert call(2, arr(4, 8), arr(8, 2), arr(0, 1)) == _hip.MG_ERR_BAD_ARG  # stride along the last axis
    assert call(2, arr(4, 8), arr(16, 1), arr(0, 1)) == _hip.MG_ERR_BAD_ARG  # an operand larger than the result
    assert call(2, arr(4, 8), arr(-8, 1), arr(0, 1)) == _hip.MG_ERR_BAD_ARG
    assert call(7, arr(*[2] * 7), arr(*[0] * 7), arr(*[0] * 7)) == _hip.MG_ERR_UNSUPPORTED
    assert call(0, arr(1), arr(0), arr(0)) == _hip.MG_ERR_UNSUPPORTED
    assert call(2, arr(1 << 16, 1 << 15), arr(0, 0), arr(0, 0)) == _hip.MG_ERR_UNSUPPORTED  # 2^31 elements
    assert call(2, arr(4, 8), arr(8, 1), arr(0, 1), dtype=2) == _hip.MG_ERR_UNSUPPORTED
    assert call(2, arr(0, 8), arr(8, 1), arr(0, 1)) == _hip.MG_OK  # nothing to do


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("sa,sb", BROADCAST_CASES)
def test_broadcasting_multiply_through_the_tensor_api(dtype, sa, sb):
    """The product is one IEEE multiply per element, so it equals NumPy's bit for bit; the
    gradient of a broadcast operand is a sum, held to the bar of the sums above."""
    import mygrad_amd as mg

    dtype = np.dtype(dtype)
    rng = np.random.default_rng([len(sa), len(sb), int(np.prod(sa)) + int(np.prod(sb))])
    av, bv = rng.standard_normal(sa).astype(dtype), rng.standard_normal(sb).astype(dtype)
    a, b = mg.Tensor(av), mg.Tensor(bv)
    out = a * b
    want = ora.multiply(av, bv)
    assert out.shape == want.shape and out.dtype == want.dtype and np.array_equal(bits(out.data), bits(want))
    g = rng.standard_normal(want.shape).astype(dtype)
    out.backward(g)
    for index, var in enumerate((a, b)):
        back = ora.multiply_broadcast_backward(g.astype(np.float64), av.astype(np.float64), bv.astype(np.float64), index)
        other = bv if index == 0 else av
        scale = ora.reduce_broadcast(np.abs(g.astype(np.float64) * other), var.shape)
        assert var.grad.shape == var.shape and var.grad.dtype == dtype
        assert np.all(np.abs(var.grad - back) <= 4 * SUM_TOL[dtype] * (scale + 1e-300))


def test_relu_gradient_uses_the_mask_of_the_forward_pass():
    """Like the reference, whose mask is made in the forward pass and kept: what x holds when
    the gradient is taken does not matter."""
    import mygrad_amd as mg
    from mygrad_amd.nnet import relu

    rng = np.random.default_rng(97)
    xv = rng.standard_normal((5, 13)).astype(np.float32)
    g = rng.standard_normal((5, 13)).astype(np.float32)
    with mg.mem_guard_off:
        x = mg.Tensor(xv.copy())
        y = relu(x)
        x.data[...] = -x.data  # allowed without the guard
        y.backward(g)
    assert np.array_equal(x.grad, ora.relu_backward(xv, g))


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

    scale = mg.Tensor([10.0, 100.0])
    prod = mg.multiply(mg.Tensor([[1.0, 2.0], [3.0, 4.0]]), scale)
    assert np.array_equal(prod.data, [[10.0, 200.0], [30.0, 400.0]])
    prod.backward()
    assert np.array_equal(scale.grad, [4.0, 6.0])
    assert np.array_equal(mg.sum(mg.Tensor([[1.0, 2.0], [3.0, 4.0]]), axis=0).data, [4.0, 6.0])
    with pytest.raises(ValueError):
        mg.multiply(mg.Tensor(np.ones((2, 3))), np.ones(4))
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
