"""Parity of ``repeat`` (forward and gradient) and of the device copy of a sliding-window
view with the NumPy restatement of the reference.

Bars: the forward pass and the window copy move bytes and are bit-exact for every dtype;
the gradient is bit-exact for unequal repeats (the reference's ``np.add.at`` adds in ascending
order in the gradient's dtype, and so does the kernel) and within 4 ulp-sized steps per added
term for equal repeats (there the reference sums a strided view in NumPy's own order)."""

import numpy as np
import pytest

from oracle import np_oracle as ora

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def abi():
    import mygrad_amd

    if not mygrad_amd.is_available():
        pytest.fail("libmygrad_hip.so / gfx950 device not available: the GPU tests need both")
    from tests import abi as module

    return module


def bits(a):
    return np.ascontiguousarray(a).view(f"u{a.dtype.itemsize}")


REPEAT_CASES = [
    ((5,), 1, None),
    ((5,), 4, 0),
    ((7, 3), 2, None),
    ((2, 3), 3, 1),
    ((2, 3, 4), 2, -2),
    ((3, 5, 8), 3, 1),  # rows of 8: 16-byte pieces
    ((4, 6, 16), 5, 0),
    ((2, 3), [1, 2], 0),
    ((2, 3), [0, 2, 5], 1),
    ((2, 2), [2, 0, 1, 3], None),
    ((3, 4, 12), [3, 0, 1, 7], 1),
    ((64, 128, 36), 2, 1),
    ((1 << 16,), 3, None),
    ((300, 40), list(range(40)), 1),
    # equal repeats along the last axis with whole 16-byte pieces: the vector kernels
    ((4, 8), 3, 1),
    ((16,), 5, None),
    ((2, 3, 64), 2, -1),
    ((32,), 1, 0),
    ((1024,), 7, None),
    ((6, 4, 12), 9, 2),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int8, np.int16, np.int32, np.int64, np.bool_])
@pytest.mark.parametrize("shape, repeats, axis", REPEAT_CASES)
def test_repeat_forward_is_bit_exact(abi, shape, repeats, axis, dtype):
    rng = np.random.default_rng([len(shape), int(np.prod(shape)), 3])
    if np.issubdtype(dtype, np.floating):
        a = rng.standard_normal(shape).astype(dtype)
        specials = np.array([np.nan, -0.0, np.inf, 0.0, -np.inf], dtype=dtype)
        a.reshape(-1)[: min(a.size, 5)] = specials[: min(a.size, 5)]
    else:
        a = rng.integers(-100, 100, shape).astype(dtype)
    got = abi.repeat_fwd(a, repeats, axis)
    want = ora.repeat_forward(a, repeats, axis)
    assert got.shape == want.shape and got.dtype == want.dtype
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape, repeats, axis", REPEAT_CASES)
def test_repeat_gradient(abi, shape, repeats, axis, dtype):
    rng = np.random.default_rng([len(shape), int(np.prod(shape)), 4])
    a = np.zeros(shape, dtype=dtype)
    out_shape = ora.repeat_forward(a, repeats, axis).shape
    grad = (rng.standard_normal(out_shape) * 10.0 ** rng.integers(-3, 4, out_shape)).astype(dtype)
    got = abi.repeat_bwd(grad, shape, repeats, axis)
    want = ora.repeat_backward(grad, a, repeats, axis)
    assert got.shape == want.shape and got.dtype == want.dtype == dtype
    if np.ndim(repeats):
        assert np.array_equal(bits(got), bits(want))  # np.add.at: ascending, in dtype, from +0.0
    else:
        exact = ora.repeat_backward(np.abs(grad).astype(np.float64), a, repeats, axis)  # sum |g| per entry
        wide = ora.repeat_backward(grad.astype(np.float64), a, repeats, axis)
        assert np.all(np.abs(got - wide) <= 4 * int(repeats) * np.finfo(dtype).eps * exact)
        assert np.all(np.abs(got - want) <= 8 * int(repeats) * np.finfo(dtype).eps * exact)


def test_repeat_reference_docstring_vectors_through_the_tensor_api(kats):
    import mygrad_amd as mg
    from mygrad_amd import _graph

    for case in kats["repeat"]:
        out = mg.repeat(mg.Tensor(case["a"]), case["repeats"], case["axis"])
        assert out.constant and out.dtype == np.array(case["a"]).dtype
        assert np.array_equal(out.data, np.array(case["out"])), case["source"]

    for shape, repeats, axis in [((), 3, None), ((), 2, 0), ((2, 3), 0, 1), ((2, 3), [0, 0, 0], 1)] + REPEAT_CASES[:11]:
        for dtype in (np.float32, np.float64):
            rng = np.random.default_rng([len(shape), int(np.prod(shape)), 6])
            x = mg.Tensor(rng.standard_normal(shape).astype(dtype))
            out = mg.repeat(x, repeats, axis)
            want = ora.repeat_forward(x.data, repeats, axis)
            assert out.shape == want.shape and out.dtype == dtype and np.array_equal(bits(out.data), bits(want))
            grad = rng.standard_normal(out.shape).astype(dtype)
            out.backward(grad)
            want_da = np.asarray(ora.repeat_backward(grad, x.data, repeats, axis)).reshape(shape)
            assert x.grad.shape == shape and x.grad.dtype == dtype
            assert np.allclose(x.grad, want_da, rtol=1e-5 if dtype == np.float32 else 1e-13, atol=1e-6 if dtype == np.float32 else 1e-14)
    assert _graph.held_count() == 0

    with pytest.raises(ValueError):
        mg.repeat(mg.Tensor(np.ones((2, 3))), [1, 2], axis=1)  # wrong number of repeats
    with pytest.raises(ValueError):
        mg.repeat(mg.Tensor(np.ones((2, 3))), -1)
    with pytest.raises(np.exceptions.AxisError):
        mg.repeat(mg.Tensor(np.ones((2, 3))), 2, axis=2)
    with pytest.raises(TypeError):
        mg.repeat(mg.Tensor(np.ones((2, 3))), np.array([1.5, 2.0]), axis=0)  # NumPy refuses the unsafe cast


WINDOW_CASES = [
    # x shape, window, step, dilation
    ((10,), (3,), (1,), (1,)),
    ((10,), (3,), (2,), (3,)),
    ((4, 9), (2,), (3,), (2,)),
    ((5, 7), (2, 3), (1, 2), (1, 1)),
    ((2, 3, 8, 9), (3, 3), (1, 1), (1, 1)),
    ((2, 3, 8, 9), (2, 3), (2, 3), (3, 2)),
    ((2, 6, 7, 8), (2, 3, 2), (1, 2, 3), (2, 1, 2)),
    ((3, 4, 32, 32), (5, 5), (2, 1), (2, 2)),
    ((2, 2, 8, 16, 16), (3, 3, 3), (1, 1, 1), (1, 1, 1)),
    ((6, 6), (6, 6), (1, 1), (1, 1)),
    ((300, 20, 37), (3, 3), (1, 1), (1, 1)),  # more planes than one block stages; 35 = 2 * 16 + 3 placements per row
    ((5, 70, 50), (3, 2), (4, 5), (1, 7)),
    ((2, 10, 10, 6), (9, 9, 3), (1, 1, 1), (1, 1, 1)),  # 81 window rows: not staged
    ((2, 40000), (9000,), (3000,), (4,)),  # a window too long for LDS
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int8, np.int16])
@pytest.mark.parametrize("shape, window, step, dilation", WINDOW_CASES)
def test_window_copy_equals_the_view(abi, shape, window, step, dilation, dtype):
    rng = np.random.default_rng([len(shape), int(np.prod(shape)), 8])
    x = (rng.standard_normal(shape) * 50).astype(dtype)
    want = np.ascontiguousarray(ora.window_view(x, window, step, dilation))
    got = abi.window_gather(x, window, step, dilation)
    assert got.shape == want.shape and np.array_equal(bits(got), bits(want))


def test_window_copy_public_function_and_errors(kats):
    import mygrad_amd as mg

    x = np.arange(36).reshape(6, 6)
    got = mg.sliding_window_copy(x, (3, 3), 3)
    view = mg.sliding_window_view(x, (3, 3), 3)
    assert got.flags["C_CONTIGUOUS"] and got.flags["WRITEABLE"] and got.dtype == x.dtype
    assert np.array_equal(got, view)
    x = np.random.default_rng(0).standard_normal((2, 3, 12, 10)).astype(np.float32)
    assert np.array_equal(mg.sliding_window_copy(x, (4, 3), (2, 1), (2, 3)), mg.sliding_window_view(x, (4, 3), (2, 1), (2, 3)))
    assert np.array_equal(mg.sliding_window_copy(x[:, :, ::2], (2, 2), 1), mg.sliding_window_view(x[:, :, ::2], (2, 2), 1))
    arrays = {"arange(36).reshape(6,6)": np.arange(36).reshape(6, 6), "arange(20).reshape(2,10)": np.arange(20).reshape(2, 10)}
    for case in kats["window"]:  # the reference's own vectors for the view
        got = mg.sliding_window_copy(arrays[case["arr"]], tuple(case["window_shape"]), tuple(case["step"]))
        if "shape" in case:
            assert list(got.shape) == case["shape"], case["source"]
        if "view" in case:
            assert np.array_equal(got, np.array(case["view"])), case["source"]
        for key, value in case.get("picks", {}).items():
            assert np.array_equal(got[tuple(int(i) for i in key.split(","))], np.array(value)), case["source"]
    with pytest.raises(ValueError):
        mg.sliding_window_copy(np.ones((3, 3)), (4, 4), 1)
    with pytest.raises(TypeError):
        mg.sliding_window_copy(np.ones((3, 3)), 2, 1)
    with pytest.raises(NotImplementedError):
        mg.sliding_window_copy(np.ones((2, 2, 2, 2)), (1, 1, 1, 1), 1)


def test_abi_rejects_bad_arguments(abi):
    from mygrad_amd import _device, _hip

    buf = _device.DeviceBuffer(4096)
    lib, p = _hip.lib(), buf.ptr
    assert lib.mg_repeat_fwd(4, 1, 4, 1, 2, 8, None, p, p + 256) == 0
    assert lib.mg_repeat_fwd(3, 1, 4, 1, 2, 8, None, p, p) == -2
    assert lib.mg_repeat_fwd(4, 1, 4, 1, 2, 9, None, p, p) == -1  # total is not n * repeats
    assert lib.mg_repeat_fwd(4, 1, 4, 1, -1, 8, None, p, p) == -1
    assert lib.mg_repeat_fwd(4, 1, 4, 1, 2, 8, None, None, p) == -1
    assert lib.mg_repeat_bwd(2, 1, 4, 1, 2, 8, None, p, p) == -2
    assert lib.mg_repeat_bwd(0, 1, 4, 1, 2, 8, None, p, None) == -1
    good = _hip.window_desc(4, 1, (10,), (3,), (1,), (1,), (8,))
    assert lib.mg_window_gather(good, p, p + 256) == 0
    assert lib.mg_window_gather(_hip.window_desc(4, 1, (10,), (3,), (1,), (1,), (9,)), p, p) == -1  # a placement too many
    assert lib.mg_window_gather(_hip.window_desc(3, 1, (10,), (3,), (1,), (1,), (8,)), p, p) == -2
    assert lib.mg_window_gather(None, p, p) == -1


# ----------------------------------------------------------------------------- transposition
PERMUTE_CASES = [
    ((5,), (0,)), ((3, 4), (1, 0)), ((3, 4), (0, 1)), ((33, 65), (1, 0)), ((2, 3, 4), (2, 0, 1)), ((2, 3, 4), (0, 2, 1)),
    ((2, 3, 4), (1, 0, 2)), ((7, 1, 5), (2, 1, 0)), ((4, 5, 6, 7), (3, 1, 0, 2)), ((4, 5, 6, 8), (1, 0, 2, 3)),
    ((2, 3, 4, 5, 6), (4, 3, 2, 1, 0)), ((2, 3, 2, 3, 2, 3), (5, 3, 1, 4, 2, 0)), ((64, 100, 36), (0, 2, 1)),
    ((100, 257), (1, 0)), ((8, 16, 12, 12), (0, 2, 3, 1)), ((8, 12, 12, 16), (0, 3, 1, 2)), ((1, 1, 1), (2, 0, 1)),
    ((300, 2, 70), (1, 2, 0)), ((1000, 1000), (1, 0)), ((3, 70000), (1, 0)), ((70000, 3), (1, 0)),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape, perm", PERMUTE_CASES)
def test_permute_is_numpys_transpose(abi, dtype, shape, perm):
    rng = np.random.default_rng([len(shape), int(np.prod(shape))])
    x = rng.standard_normal(shape).astype(dtype)
    got = abi.permute(x, perm)
    want = np.ascontiguousarray(np.transpose(x, perm))
    assert got.shape == want.shape and np.array_equal(got.view(np.uint8), want.view(np.uint8))


def test_permute_rejects_bad_arguments(abi):
    import ctypes

    from mygrad_amd import _device, _hip

    buf = _device.DeviceBuffer(256)
    lib = _hip.lib()
    shape, perm = (ctypes.c_int64 * 2)(3, 4), (ctypes.c_int32 * 2)(1, 1)
    assert lib.mg_permute(4, 2, shape, perm, buf.ptr, buf.ptr) == _hip.MG_ERR_BAD_ARG  # not a permutation
    perm = (ctypes.c_int32 * 2)(1, 0)
    assert lib.mg_permute(2, 2, shape, perm, buf.ptr, buf.ptr) == _hip.MG_ERR_UNSUPPORTED  # 2-byte elements
    assert lib.mg_permute(4, 2, shape, perm, None, buf.ptr) == _hip.MG_ERR_BAD_ARG
    seven = (ctypes.c_int64 * 7)(*([2] * 7))
    reverse = (ctypes.c_int32 * 7)(*range(6, -1, -1))
    assert lib.mg_permute(4, 7, seven, reverse, buf.ptr, buf.ptr) == _hip.MG_ERR_UNSUPPORTED  # seven axes that all move


# ----------------------------------------------------------------------------- strided copy
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_strided_copy_walks_diagonals_both_ways(abi, dtype):
    rng = np.random.default_rng(91)
    x = rng.standard_normal((5, 7, 5)).astype(dtype)
    # the diagonal over axes 0 and 2, laid out (i, j): strides (35 + 1, 5)
    got = abi.strided_copy(x, (5, 7), (36, 5))
    assert np.array_equal(got, np.einsum("iji->ij", x))
    back = abi.strided_copy(got, (5, 7), (36, 5), out_elems=x.size).reshape(x.shape)
    want = np.zeros_like(x)
    i = np.arange(5)
    want[i, :, i] = got
    assert np.array_equal(back, want)
    # a plain transposition is the same call
    y = rng.standard_normal((30, 41)).astype(dtype)
    assert np.array_equal(abi.strided_copy(y, (41, 30), (1, 41)), y.T)


def test_strided_copy_rejects_what_would_leave_the_buffer(abi):
    import ctypes

    from mygrad_amd import _device, _hip

    buf = _device.DeviceBuffer(4096)
    lib = _hip.lib()
    shape, strides = (ctypes.c_int64 * 2)(4, 4), (ctypes.c_int64 * 2)(5, 1)
    assert lib.mg_strided_copy(4, 2, shape, strides, 19, 0, buf.ptr, buf.ptr) == _hip.MG_OK  # reaches element 3*5 + 3 = 18
    assert lib.mg_strided_copy(4, 2, shape, strides, 18, 0, buf.ptr, buf.ptr) == _hip.MG_ERR_BAD_ARG
    negative = (ctypes.c_int64 * 2)(5, -1)
    assert lib.mg_strided_copy(4, 2, shape, negative, 64, 0, buf.ptr, buf.ptr) == _hip.MG_ERR_BAD_ARG
    assert lib.mg_strided_copy(2, 2, shape, strides, 64, 0, buf.ptr, buf.ptr) == _hip.MG_ERR_UNSUPPORTED


def test_permute_full_size_round_trip(abi):
    """The benchmark's tensor (134 MB): channels last and back gives the input, bit for bit."""
    rng = np.random.default_rng(93)
    x = rng.standard_normal((8, 32, 32, 64, 64), dtype=np.float32)
    there = abi.permute(x, (0, 2, 3, 4, 1))
    assert np.array_equal(there[3, 5, 7, 11], x[3, :, 5, 7, 11])
    assert np.array_equal(abi.permute(there, (0, 4, 1, 2, 3)), x)
