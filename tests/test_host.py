"""Host-side logic that needs no GPU: the C-ABI library loads and exports what
the header declares, argument validation raises the reference's exception types
before anything is launched, the window helper, and the graph semantics of the
Tensor / Operation shim (exercised with a tiny NumPy-only operation defined
here)."""

import ctypes
import os
import re

import numpy as np
import pytest

import mygrad_amd as mg
from mygrad_amd import _graph, _hip
from mygrad_amd.nnet import conv_nd, max_pool

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ----------------------------------------------------------------------------- C ABI
def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mygrad_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mg_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _hip.load_library()
    declared = _declared_symbols()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in mygrad_hip.h but not exported"
    assert sorted(_hip.EXPORTED_SYMBOLS) == declared


def test_struct_layouts_match_header():
    # int32 x2 + int64 x3 + 6 * int64[3]
    assert ctypes.sizeof(_hip.ConvDesc) == 8 + 24 + 6 * 24
    assert ctypes.sizeof(_hip.PoolDesc) == 16 + 8 + 4 * 24
    assert ctypes.sizeof(_hip.DeviceInfo) == 64 + 16 + 8 + 16
    assert ctypes.sizeof(_hip.BnDesc) == 16 + 24 + 8
    assert ctypes.sizeof(_hip.WindowDesc) == 8 + 8 + 5 * 24


def test_calls_before_init_report_not_initialised():
    if _hip._ready:
        pytest.skip("a device is initialised in this process")
    lib = _hip.load_library()
    assert lib.mg_sync() == _hip.MG_ERR_NOT_INIT
    assert "mg_init" in _hip.last_error()
    ptr = ctypes.c_void_p()
    assert lib.mg_malloc(ctypes.byref(ptr), 16) == _hip.MG_ERR_NOT_INIT


def test_no_device_fails_loudly_without_fallback():
    if mg.is_available():
        pytest.skip("a GPU is present")
    x = np.zeros((1, 1, 4, 4))
    with pytest.raises(mg.HipUnavailable):
        conv_nd(x, np.zeros((1, 1, 2, 2)), stride=1)
    with pytest.raises(mg.HipUnavailable):
        max_pool(x, (2, 2), 2)
    assert _graph.held_count() == 0  # a failing op releases its locks
    assert x.flags.writeable
    # and so do the operations either side of them
    from mygrad_amd.nnet import batchnorm, relu

    v = np.ones((2, 3))
    for call in (
        lambda: relu(v),
        lambda: mg.multiply(v, v),
        lambda: mg.sum(v),
        lambda: batchnorm(v, eps=1e-5),
        lambda: mg.repeat(v, 2),
        lambda: mg.matmul(v, v.T),
        lambda: mg.Tensor(v) @ v.T,
        lambda: mg.sliding_window_copy(v, (2, 2), 1),
        lambda: mg.sum(v, axis=0),
        lambda: mg.multiply(v, np.ones(3)),
        lambda: mg.einsum("ij,kj->ik", v, v),
        lambda: mg.einsum("ij->ji", v),
    ):
        with pytest.raises(mg.HipUnavailable):
            call()
    assert _graph.held_count() == 0


# ----------------------------------------------------------------------------- validation (no launch)
@pytest.mark.parametrize(
    "x_shape,w_shape",
    [((4,), (1, 1, 2)), ((3, 3), (1, 3, 2)), ((1, 2, 5), (1, 2)), ((1, 2, 5, 5), (1, 2, 3)), ((1, 2, 5), (1, 3, 2))],
)
def test_conv_shape_mismatch_is_value_error(x_shape, w_shape):
    with pytest.raises(ValueError):
        conv_nd(np.zeros(x_shape), np.zeros(w_shape), stride=1)


def test_conv_error_contract():
    x = np.zeros((1, 2, 2, 2))
    w = np.zeros((1, 2, 2, 2))
    with pytest.raises(ValueError):
        conv_nd(x, np.zeros((1, 3, 2, 2)), stride=1, padding=0)  # mismatched channels
    with pytest.raises(ValueError):
        conv_nd(x, np.zeros((1, 2, 3, 2)), stride=1, padding=0)  # filter larger than data
    with pytest.raises(AssertionError):
        conv_nd(x, w, stride=0, padding=0)
    with pytest.raises(AssertionError):
        conv_nd(x, w, stride=[1, 2, 3])
    with pytest.raises(AssertionError):
        conv_nd(x, w, stride=1, padding=-1)
    with pytest.raises(AssertionError):
        conv_nd(x, w, stride=1, padding=[1, 2, 3])
    with pytest.raises(AssertionError):
        conv_nd(x, w, stride=1, dilation=0)
    with pytest.raises(ValueError) as info:
        conv_nd(x, w, stride=3, padding=1)  # non-integer output extent
    assert "Stride and kernel dimensions are incompatible" in str(info.value)
    # the benchmark shapes the reference rejects are rejected here too
    with pytest.raises(ValueError):
        conv_nd(np.zeros((1, 1, 28, 28), np.float32), np.zeros((1, 1, 3, 3), np.float32), stride=2, padding=1)
    # the window helper's w*d <= extent rule, applied to the padded data
    with pytest.raises(ValueError):
        conv_nd(np.zeros((1, 1, 3)), np.zeros((1, 1, 2)), stride=1, dilation=2)
    assert _graph.held_count() == 0 and x.flags.writeable and w.flags.writeable


def test_pool_error_contract():
    x = mg.Tensor(np.zeros((1, 2, 2, 2)), dtype="float32")
    with pytest.raises(ValueError):
        max_pool(x, (3,) * 3, (1,) * 3)
    with pytest.raises(AssertionError):
        max_pool(x, (2,) * 3, (0,) * 3)
    with pytest.raises(AssertionError):
        max_pool(x, (2,) * 2, [1, 2, 3])
    with pytest.raises(AssertionError):
        max_pool(x, 2, 1)  # pool must be a sequence
    with pytest.raises(AssertionError):
        max_pool(x, (2, 0), 1)
    with pytest.raises(ValueError) as info:
        max_pool(x, (1,) * 3, (3,) * 3)
    assert "Pooling dimensions" in str(info.value)
    with pytest.raises(ValueError):
        max_pool(np.zeros((1, 1, 56, 56)), (3, 3), 2)  # 27.5 placements
    assert _graph.held_count() == 0


def test_unsupported_inputs_are_rejected_not_computed_on_the_cpu():
    with pytest.raises(TypeError):
        conv_nd(np.zeros((1, 1, 4), np.complex64), np.zeros((1, 1, 2), np.complex64), stride=1)
    with pytest.raises(TypeError):
        max_pool(np.zeros((1, 4), bool), (2,), 2)
    # integers run as float64, which is exact below 2**53 only
    with pytest.raises(TypeError):
        max_pool(np.full((1, 4), 2**60), (2,), 2)
    with pytest.raises(TypeError):
        conv_nd(np.full((1, 1, 4), 2**30), np.full((1, 1, 2), 2**30), stride=1)
    with pytest.raises(NotImplementedError):
        max_pool(np.zeros((4, 4)), (), ())  # nothing to pool over


# ----------------------------------------------------------------------------- window helper
def test_sliding_window_view_vectors(kats):
    case = kats["window"][0]
    y = mg.sliding_window_view(np.arange(36).reshape(6, 6), window_shape=case["window_shape"], step=case["step"])
    assert list(y.shape) == case["shape"]
    for key, want in case["picks"].items():
        i, j = map(int, key.split(","))
        assert np.array_equal(y[i, j], np.array(want))
    want = np.array(kats["window"][1]["view"])
    x = np.asfortranarray(np.arange(20).reshape(2, 10))
    y = mg.sliding_window_view(x, (5,), 5)
    assert not y.flags.writeable and np.array_equal(y, want)
    x = np.arange(20).reshape(2, 10)
    y = mg.sliding_window_view(x, (5,), 5)
    assert np.shares_memory(x, y) and np.array_equal(y, want)


def test_sliding_window_view_matches_slicing():
    rng = np.random.default_rng(3)
    for _ in range(200):
        nd = int(rng.integers(1, 5))
        shape = tuple(int(v) for v in rng.integers(1, 8, nd))
        x = rng.integers(0, 100, shape)
        m = int(rng.integers(1, nd + 1))
        tail = shape[-m:]
        win = tuple(int(rng.integers(1, s + 1)) for s in tail)
        step = tuple(int(rng.integers(1, s + 1)) for s in tail)
        dil = tuple(int(rng.integers(1, s // w + 1)) for s, w in zip(tail, win))
        y = mg.sliding_window_view(x, win, step, dil)
        for g in np.ndindex(*y.shape[:m]):
            sl = tuple(slice(i * s, i * s + w * d, d) for i, w, s, d in zip(g, win, step, dil))
            assert np.array_equal(y[g], x[(Ellipsis, *sl)])


@pytest.mark.parametrize(
    "kwargs",
    [dict(step=None), dict(step=-1), dict(window_shape=None), dict(window_shape=1), dict(window_shape=(1, 1, 1)),
     dict(window_shape=(-1, 1)), dict(window_shape=(1.0, 2.0)), dict(window_shape=(7, 5)), dict(dilation=-1),
     dict(dilation=(1, 0)), dict(dilation="aa"), dict(dilation=(1, 1, 1)), dict(dilation=1.0), dict(dilation=7),
     dict(dilation=(1, 7)), dict(dilation=(10, 1))],
)
def test_sliding_window_view_validation(kwargs):
    args = dict(arr=np.arange(36).reshape(6, 6), window_shape=(1, 1), step=1, dilation=None)
    args.update(kwargs)
    with pytest.raises((ValueError, TypeError)):
        mg.sliding_window_view(**args)


# ----------------------------------------------------------------------------- graph semantics
class Scale(mg.Operation):
    """out = a * x + b * y, a NumPy-only stand-in used to drive the shim."""

    def __call__(self, x, y, a=2.0, b=3.0):
        self.variables = (x, y)
        self.a, self.b = a, b
        return a * x.data + b * y.data

    def backward_var(self, grad, index, **kwargs):
        return (self.a if index == 0 else self.b) * grad


class Identity(mg.Operation):
    def __call__(self, x):
        self.variables = (x,)
        return x.data.copy()

    def backward_var(self, grad, index, **kwargs):
        return grad  # the incoming gradient itself: the caller must copy it


def test_op_wraps_output_without_copy_and_locks_arrays():
    x = mg.Tensor([1.0, 2.0])
    y = np.array([3.0, 4.0])
    captured = {}

    class Spy(Scale):
        def __call__(self, *a, **k):
            captured["out"] = super().__call__(*a, **k)
            return captured["out"]

    out = mg.execute_op(Spy, x, y)
    assert out.data is captured["out"]
    assert isinstance(out.creator, Spy) and out.creator.variables[0] is x
    assert out.creator.variables[1].data is y and out.creator.variables[1].constant
    assert not x.data.flags.writeable and not y.flags.writeable and not out.data.flags.writeable
    out.backward()
    assert x.data.flags.writeable and y.flags.writeable and out.data.flags.writeable
    assert out.creator is None and _graph.held_count() == 0
    assert np.array_equal(x.grad, [2.0, 2.0])


class _HostBackedBuffer:
    """Stands in for a device buffer in the tests of the host logic: 'downloads' from a NumPy array."""

    def __init__(self, values):
        self.values = np.ascontiguousarray(values)
        self.ptr, self.nbytes, self.downloads = 0, self.values.nbytes, 0

    def download_into(self, arr):
        self.downloads += 1
        arr[...] = self.values.reshape(arr.shape)


def _pinned_stand_in(monkeypatch):
    from mygrad_amd import _device

    monkeypatch.setattr(_device, "pinned_empty", lambda shape, dtype: np.empty(shape, dtype))
    return _device


class DeviceScale(mg.Operation):
    """Doubles its input and returns the result as a value that is 'on the device' only."""

    takes_device_arrays = True

    def __call__(self, x):
        from mygrad_amd import _device

        self.variables = (x,)
        self.seen = _device.value_of(x)
        values = np.asarray(self.seen.buf.values if isinstance(self.seen, _device.DeviceArray) else self.seen) * 2.0
        return _device.DeviceArray(_HostBackedBuffer(values), values.shape, values.dtype)

    def backward_var(self, grad, index, **kwargs):
        from mygrad_amd import _device

        self.grad_seen = grad
        values = np.asarray(grad.buf.values if isinstance(grad, _device.DeviceArray) else grad) * 2.0
        return _device.DeviceArray(_HostBackedBuffer(values), values.shape, values.dtype)


def test_a_result_on_the_device_is_copied_once_when_read_and_guarded_like_any_array(monkeypatch):
    _device = _pinned_stand_in(monkeypatch)
    x = mg.Tensor([1.0, 2.0, 3.0])
    y = mg.execute_op(DeviceScale, x)
    z = mg.execute_op(DeviceScale, y)
    assert y.on_device and z.on_device and y.shape == (3,) and y.dtype == np.float64 and y.size == 3 and y.ndim == 1
    assert isinstance(z.creator.seen, _device.DeviceArray)  # the second operation got the value as it was, no copy
    buf = y._value.buf
    data = y.data
    assert buf.downloads == 1 and y.data is data and not y.on_device
    assert np.array_equal(data, [2.0, 4.0, 6.0])
    assert not data.flags.writeable  # two live operations hold it (its creator and its consumer)
    z.backward(np.array([1.0, 1.0, 1.0]))
    assert data.flags.writeable and _graph.held_count() == 0
    assert isinstance(x._grad, _device.DeviceArray)  # a gradient stays where it was made ...
    grad = x.grad
    assert isinstance(grad, np.ndarray) and np.array_equal(grad, [4.0, 4.0, 4.0]) and x.grad is grad  # ... until it is read
    assert grad.flags.writeable
    # read after its graph is gone: an ordinary writeable array, nothing left to guard
    w = mg.execute_op(DeviceScale, x)
    w.clear_graph()
    assert w.data.flags.writeable
    # without the graph (or the guard) nothing is locked and nothing is remembered
    with mg.no_autodiff:
        v = mg.execute_op(DeviceScale, x)
    assert v.on_device and v.creator is None and v.data.flags.writeable
    assert _graph.held_count() == 0


def test_an_operation_that_does_not_take_device_arrays_gets_host_arrays(monkeypatch):
    _device = _pinned_stand_in(monkeypatch)
    x = mg.Tensor([1.0, 2.0])
    y = mg.execute_op(DeviceScale, x)
    out = mg.execute_op(Scale, y, np.array([1.0, 1.0]))  # reads y.data: a host array from here on
    assert not y.on_device and np.array_equal(out.data, [7.0, 11.0])
    out.backward()
    assert np.array_equal(x.grad, [4.0, 4.0])
    u = mg.Tensor([1.0, 2.0])
    z = mg.execute_op(DeviceScale, mg.execute_op(Identity, u))
    z.backward(np.array([1.0, 1.0]))  # DeviceScale hands a DeviceArray back; Identity's backward_var gets an ndarray
    assert isinstance(z.creator, type(None)) and np.array_equal(u.grad, [2.0, 2.0])
    assert _graph.held_count() == 0


def test_device_array_answers_shape_questions_without_a_copy():
    from mygrad_amd import _device

    buf = _HostBackedBuffer(np.arange(24.0))
    a = _device.DeviceArray(buf, (2, 3, 4), np.float64)
    assert (a.ndim, a.size, a.nbytes, a.itemsize) == (3, 24, 192, 8) and a.flags["C_CONTIGUOUS"] and a.base is None
    b = a.reshape(6, -1)
    assert b.shape == (6, 4) and b.buf is buf and b.base is a and b.reshape((24,)).base is a
    with pytest.raises(ValueError):
        a.reshape(5, -1)
    assert buf.downloads == 0 and _device.is_locked(a) and _device.lookup(a) is buf


def test_constant_propagation():
    f, c = mg.Tensor([1.0]), mg.Tensor([1.0], constant=True)
    assert mg.execute_op(Scale, f, c).constant is False
    assert mg.execute_op(Scale, c, c).constant is True
    assert mg.execute_op(Scale, f, f, constant=True).constant is True
    assert mg.execute_op(Scale, c, [1.0]).constant is True
    assert mg.Tensor([1, 2]).constant is True
    with pytest.raises(ValueError):
        mg.Tensor([1, 2], constant=False)
    with pytest.raises(TypeError):
        mg.Tensor([1.0], constant="yes")
    out = mg.execute_op(Scale, c, c)
    out.backward()  # constant terminal: clears the graph, computes nothing
    assert c.grad is None and out.grad is None and _graph.held_count() == 0
    for t in (f,):
        t.clear_graph()


def test_backward_seed_accumulation_dtype_and_aliasing():
    x = mg.Tensor(np.array([1.0, 2.0, 3.0], dtype=np.float32))
    out = mg.execute_op(Scale, x, x)  # x feeds the op twice: 2*g then += 3*g
    g = np.array([1.0, 10.0, 100.0])
    out.backward(g)
    assert x.grad.dtype == np.float32
    assert np.array_equal(x.grad, 5 * g.astype(np.float32))
    assert np.array_equal(g, [1.0, 10.0, 100.0]) and out.grad.dtype == np.float32
    assert out.grad is not g

    x = mg.Tensor([1.0, 2.0])
    out = mg.execute_op(Identity, x)
    out.backward()
    assert x.grad is not out.grad and not np.shares_memory(x.grad, out.grad)
    out2 = mg.execute_op(Identity, x)  # entering a new graph nulls the old gradient
    assert x.grad is None
    out2.backward(2.0)  # broadcast seed
    assert np.array_equal(x.grad, [2.0, 2.0])
    with pytest.raises(ValueError):
        mg.execute_op(Identity, x).backward(np.ones(3))
    x.clear_graph()


def test_invalid_gradient_and_cleared_graph():
    class Bad(Identity):
        def backward_var(self, grad, index, **kwargs):
            return "not an array"

    x = mg.Tensor([1.0])
    with pytest.raises(mg.InvalidGradient):
        mg.execute_op(Bad, x).backward()
    x.clear_graph()

    x = mg.Tensor([1.0])
    mid = mg.execute_op(Identity, x)
    out = mg.execute_op(Identity, mid)
    x._ops.clear()  # what clearing the upstream part of the graph leaves behind
    with pytest.raises(mg.InvalidBackprop):
        out.backward()
    out.clear_graph()


def test_chain_and_fan_out_topological_order():
    x = mg.Tensor([1.0, 2.0])
    a = mg.execute_op(Scale, x, x, op_kwargs=dict(a=1.0, b=1.0))  # 2x
    b = mg.execute_op(Scale, a, x, op_kwargs=dict(a=1.0, b=1.0))  # 3x
    c = mg.execute_op(Scale, a, b, op_kwargs=dict(a=1.0, b=1.0))  # 5x
    c.backward()
    assert np.array_equal(x.grad, [5.0, 5.0]) and np.array_equal(a.grad, [2.0, 2.0])
    assert _graph.held_count() == 0


def test_no_autodiff_and_mem_guard_switches():
    x = mg.Tensor([1.0])
    with mg.no_autodiff:
        out = mg.execute_op(Identity, x)
        assert out.creator is None and x.data.flags.writeable
        out.backward()  # no-op
    assert x.grad is None

    @mg.no_autodiff
    def run(t):
        return mg.execute_op(Identity, t)

    assert run(x).creator is None and _graph.TRACK_GRAPH is True
    with mg.mem_guard_off:
        out = mg.execute_op(Identity, x)
        assert x.data.flags.writeable and out.creator is not None
        out.backward()
    assert np.array_equal(x.grad, [1.0])


def test_save_and_load_round_trip(tmp_path):
    import io

    import mygrad_amd as mg

    x = mg.Tensor(np.arange(10.0))
    buf = io.BytesIO()
    mg.save(buf, x)
    buf.seek(0)
    back = mg.load(buf)
    assert isinstance(back, mg.Tensor) and np.array_equal(back.data, x.data) and back.grad is None

    x.backward(np.arange(10.0) * 2)  # a leaf: the seed becomes its gradient
    path = tmp_path / "with_grad"
    mg.save(path, x)
    back = mg.load(str(path) + ".npz")
    assert np.array_equal(back.data, x.data) and np.array_equal(back.grad, np.arange(10.0) * 2)
    with np.load(str(path) + ".npz") as archive:  # the reference's layout
        assert sorted(archive.files) == ["data", "grad"]

    ints = mg.Tensor(np.arange(4))
    buf = io.BytesIO()
    mg.save(buf, ints)
    buf.seek(0)
    assert mg.load(buf).dtype == ints.dtype
    with pytest.raises(TypeError):
        mg.save(io.BytesIO(), np.arange(3.0))


def test_argument_checks_of_the_neighbouring_operations_need_no_device():
    """Everything that is refused is refused before a kernel could be launched, with NumPy's /
    the reference's exception types; empty results are answered on the host."""
    from mygrad_amd.nnet import batchnorm

    x = np.ones((4, 3, 5))
    with pytest.raises(ValueError):
        batchnorm(np.ones(4), eps=1e-5)  # fewer than two axes
    with pytest.raises(ValueError):
        batchnorm(x, gamma=np.ones(2), eps=1e-5)
    with pytest.raises(TypeError):
        batchnorm(x.astype(np.float32), gamma=np.ones(3), eps=1e-5)  # gamma in another dtype
    with pytest.raises(TypeError):
        batchnorm(np.ones((4, 3), dtype=np.int32), eps=1e-5)
    with pytest.raises(ValueError):
        batchnorm(x, eps=-1.0)
    assert batchnorm(np.ones((0, 3, 5)), eps=1e-5).shape == (0, 3, 5)

    with pytest.raises(ValueError):
        mg.matmul(x, 3.0)  # scalars are not allowed
    with pytest.raises(ValueError):
        mg.matmul(np.ones((2, 3)), np.ones((4, 2)))
    with pytest.raises(ValueError):
        mg.matmul(np.ones((2, 1, 3, 4)), np.ones((3, 2, 4, 5)))  # stacks that do not broadcast against each other
    with pytest.raises(TypeError):
        mg.matmul(np.ones((2, 3), dtype=np.int64), np.ones((3, 2), dtype=np.int64))
    assert mg.matmul(np.ones((0, 3)), np.ones((3, 2))).shape == (0, 2)
    assert np.array_equal(mg.matmul(np.ones((2, 0)), np.ones((0, 3))).data, np.zeros((2, 3)))

    with pytest.raises(ValueError):
        mg.repeat(np.ones((2, 3)), [1, 2], axis=1)
    with pytest.raises(ValueError):
        mg.repeat(np.ones((2, 3)), -1)
    with pytest.raises(np.exceptions.AxisError):
        mg.repeat(np.ones((2, 3)), 2, axis=2)
    with pytest.raises(TypeError):
        mg.repeat(np.ones(3, dtype=np.complex128), 2)  # 16-byte elements
    assert mg.repeat(np.ones((2, 3)), 0, axis=1).shape == (2, 0)
    assert mg.repeat(np.ones((0, 3)), 2, axis=0).shape == (0, 3)

    with pytest.raises(ValueError):
        mg.sliding_window_copy(np.ones((3, 3)), (4, 4), 1)
    with pytest.raises(TypeError):
        mg.sliding_window_copy(np.ones((3, 3)), 2, 1)
    with pytest.raises(NotImplementedError):
        mg.sliding_window_copy(np.ones((2, 2, 2, 2)), (1, 1, 1, 1), 1)

    with pytest.raises(ValueError):
        mg.einsum("ij,jk->ik", np.ones((2, 3)), np.ones((4, 4)))
    with pytest.raises(ValueError):
        mg.einsum("ij,jk->ii", np.ones((2, 3)), np.ones((3, 4)))
    with pytest.raises(ValueError):
        mg.einsum("ii", np.ones((3, 4)))
    with pytest.raises(TypeError):
        mg.einsum("i,i", np.arange(3), np.arange(3))
    assert mg.einsum("ij,jk->ik", np.ones((2, 0)), np.ones((0, 3))).shape == (2, 3)
    # the target of out=, checked like np.einsum checks it, before anything is computed
    ab = (np.ones((2, 3)), np.ones((3, 4)))
    with pytest.raises(TypeError):
        mg.einsum("ij,jk->ik", *ab, out=[[0.0] * 4] * 2)
    with pytest.raises(TypeError):
        mg.einsum("ij,jk->ik", *ab, out=np.zeros((2, 4), dtype=np.float32))  # float64 into float32 is no safe cast
    with pytest.raises(ValueError):
        mg.einsum("ij,jk->ik", *ab, out=np.zeros((2, 5)))
    with pytest.raises(ValueError):
        mg.einsum("ij,jk->ik", *ab, out=np.zeros((1, 2, 4)))
    locked = np.zeros((2, 4))
    locked.flags.writeable = False
    with pytest.raises(ValueError):
        mg.einsum("ij,jk->ik", *ab, out=locked)
    with pytest.raises(NotImplementedError):
        mg.einsum("ij,jk->ik", *ab, out=mg.Tensor(np.zeros((2, 4))))  # in-place semantics on tensors
    with pytest.raises(ValueError):
        mg.einsum("ii,ij->j", np.ones((3, 1)), np.ones((3, 2)))  # a diagonal whose axes differ in length

    with pytest.raises(ValueError):
        mg.multiply(np.ones((2, 3)), np.ones(4))  # shapes that do not broadcast
    with pytest.raises(TypeError):
        mg.multiply(np.ones((2, 3), dtype=np.int64), np.ones(3, dtype=np.int64))
    assert mg.multiply(np.ones((0, 3)), np.ones(3)).shape == (0, 3)
    with pytest.raises(np.exceptions.AxisError):
        mg.sum(np.ones((2, 3)), axis=2)
    with pytest.raises(ValueError):
        mg.sum(np.ones((2, 3)), axis=(1, 1))
    with pytest.raises(TypeError):
        mg.sum(np.ones((2, 3), dtype=np.int32), axis=0)
    assert np.array_equal(mg.sum(np.ones((0, 3)), axis=0).data, np.zeros(3))
    assert mg.sum(np.ones((0, 3)), axis=1, keepdims=True).shape == (0, 1)
    assert _graph.held_count() == 0


def test_multi_matmul_picks_the_cheapest_order_and_checks_its_arguments():
    from mygrad_amd.math.misc.funcs import _chain_split

    def cheapest(dims, i, j):
        if i == j:
            return 0
        return min(cheapest(dims, i, k) + cheapest(dims, k + 1, j) + dims[i] * dims[k + 1] * dims[j + 1] for k in range(i, j))

    def cost_of(cut, dims, i, j):
        if i == j:
            return 0
        k = cut[i][j]
        return cost_of(cut, dims, i, k) + cost_of(cut, dims, k + 1, j) + dims[i] * dims[k + 1] * dims[j + 1]

    # the textbook case: A 10x100, B 100x5, C 5x50 -> (A B) C at 7500 multiplications, not 75000
    assert cost_of(_chain_split([10, 100, 5, 50]), [10, 100, 5, 50], 0, 2) == 7500
    rng = np.random.default_rng(3)
    for n in range(2, 8):
        for _ in range(10):
            dims = [int(v) for v in rng.integers(1, 30, n + 1)]
            assert cost_of(_chain_split(dims), dims, 0, n - 1) == cheapest(dims, 0, n - 1)
    with pytest.raises(ValueError):
        mg.multi_matmul([np.ones((2, 2))])
    with pytest.raises(ValueError):
        mg.multi_matmul([np.ones((2, 2)), np.ones((2, 2, 2)), np.ones((2, 2))])
    with pytest.raises(ValueError):
        mg.multi_matmul([np.ones((2, 3)), np.ones(3), np.ones((3, 2))])  # a vector in the middle


@pytest.mark.parametrize(
    "sa,sb",
    [((4, 5), (5,)), ((4, 5), (4, 1)), ((3, 1, 2), (1, 4, 1)), ((2, 3), ()), ((1,), (2, 3)), ((8, 16, 12, 12), (16, 1, 1)),
     ((2, 1, 3, 1, 2), (3, 1, 4, 1)), ((1, 1), (1,)), ((2, 1, 2, 1, 2, 1, 2), (1, 3, 1, 3, 1, 3, 1)), ((2, 3, 4), (2, 3, 4))],
)
def test_multiply_plan_reads_each_operand_where_it_lies(sa, sb):
    """The merged axes and strides of the one-pass broadcasting product, walked with NumPy's
    own strided views, give NumPy's product."""
    from numpy.lib.stride_tricks import as_strided

    from mygrad_amd import _reduce

    rng = np.random.default_rng(len(sa) * 10 + len(sb))
    a, b = rng.standard_normal(sa), rng.standard_normal(sb)
    shape = np.broadcast_shapes(sa, sb)
    extents, a_strides, b_strides = _reduce.multiply_plan(sa, sb, shape)
    assert int(np.prod(extents)) == int(np.prod(shape)) and a_strides[-1] in (0, 1) and b_strides[-1] in (0, 1)
    assert all(x > 1 for x in extents) or extents == [1]
    va = as_strided(a.reshape(-1) if a.size else a, shape=extents, strides=[8 * s for s in a_strides], writeable=False)
    vb = as_strided(b.reshape(-1) if b.size else b, shape=extents, strides=[8 * s for s in b_strides], writeable=False)
    assert np.array_equal((va * vb).reshape(shape), a * b)


def test_multiply_plan_on_drawn_shapes():
    """The same property on shapes drawn by hypothesis: any two shapes that broadcast."""
    from hypothesis import given, settings
    from hypothesis import strategies as st
    from numpy.lib.stride_tricks import as_strided

    from mygrad_amd import _reduce

    @st.composite
    def pairs(draw):
        full = draw(st.lists(st.integers(1, 4), min_size=0, max_size=7))
        def operand():
            keep = draw(st.integers(0, len(full)))
            tail = full[len(full) - keep:]
            return tuple(n if draw(st.booleans()) else 1 for n in tail)
        return operand(), operand()

    @settings(max_examples=300, deadline=None)
    @given(pairs())
    def check(pair):
        sa, sb = pair
        shape = np.broadcast_shapes(sa, sb)
        a = np.arange(1, 1 + int(np.prod(sa)), dtype=np.float64).reshape(sa)
        b = np.arange(2, 2 + int(np.prod(sb)), dtype=np.float64).reshape(sb) * 0.5
        extents, a_strides, b_strides = _reduce.multiply_plan(sa, sb, shape)
        assert int(np.prod(extents)) == int(np.prod(shape))
        assert 1 + sum((n - 1) * s for n, s in zip(extents, a_strides)) == a.size  # reaches a's last element, no further
        assert 1 + sum((n - 1) * s for n, s in zip(extents, b_strides)) == b.size
        va = as_strided(a.reshape(-1), shape=extents, strides=[8 * s for s in a_strides], writeable=False)
        vb = as_strided(b.reshape(-1), shape=extents, strides=[8 * s for s in b_strides], writeable=False)
        assert np.array_equal((va * vb).reshape(shape), a * b)

    check()


def test_pooling_stages_cover_any_number_of_axes():
    """Stage planning of max_pool over more axes than the kernels take (host logic only): every
    stage has at most three axes, each stage reads what the one before it wrote, and the last
    one's windows are the windows of the whole pooling."""
    from mygrad_amd.nnet.layers.pooling import plan_stages

    rng = np.random.default_rng(5)
    for m in range(1, 9):
        pool = rng.integers(1, 4, m)
        stride = rng.integers(1, 4, m)
        grid = rng.integers(1, 4, m)
        pooled = (grid - 1) * stride + pool
        lead = int(rng.integers(1, 5))
        stages = plan_stages(lead, pooled, pool, stride)
        assert all(1 <= len(st.shape) <= 3 for st in stages)
        assert len(stages) == (1 if m <= 3 else 1 + -(-(m - 3) // 2))
        assert stages[0].count == lead * int(np.prod(pooled))
        for before, after in zip(stages, stages[1:]):
            assert after.count == before.windows  # a stage reads exactly what the one before it wrote
        assert stages[-1].windows == lead * int(np.prod(grid))
        # window volumes multiply up to the whole window
        assert int(np.prod([np.prod(st.pool) for st in stages])) == int(np.prod(pool))


def test_shared_descriptors_are_built_once_per_distinct_layer():
    """``_hip.shared_desc`` hands the same descriptor object to every call with the same
    arguments (the operations describe the same layer at every step), builds a fresh one for
    arguments that do not hash, and never confuses two builders or two sets of settings."""
    f32, f64 = np.dtype(np.float32), np.dtype(np.float64)
    a = _hip.shared_desc(_hip.pool_desc, f32, 6, (8, 8), (2, 2), (2, 2), (4, 4), dx_dtype=None)
    b = _hip.shared_desc(_hip.pool_desc, f32, 6, (8, 8), (2, 2), (2, 2), (4, 4), dx_dtype=None)
    assert a is b
    wide = _hip.shared_desc(_hip.pool_desc, f32, 6, (8, 8), (2, 2), (2, 2), (4, 4), dx_dtype=f64)
    assert wide is not a and wide.dx_dtype == _hip.MG_F64 and a.dx_dtype == _hip.MG_F32
    other = _hip.shared_desc(_hip.pool_desc, f32, 7, (8, 8), (2, 2), (2, 2), (4, 4), dx_dtype=None)
    assert other is not a and other.lead == 7 and a.lead == 6
    listed = _hip.shared_desc(_hip.pool_desc, f32, 6, [8, 8], [2, 2], [2, 2], [4, 4])
    assert listed is not a and list(listed.X) == list(a.X) and list(listed.G) == list(a.G)
    c = _hip.shared_desc(_hip.conv_desc, f64, (2, 3, 8, 8), (4, 3, 3, 3), (8, 8), (1, 1), (1, 1), (1, 1))
    assert c is _hip.shared_desc(_hip.conv_desc, f64, (2, 3, 8, 8), (4, 3, 3, 3), (8, 8), (1, 1), (1, 1), (1, 1))
    assert (c.N, c.C, c.F, list(c.pad)) == (2, 3, 4, [0, 1, 1])
    fresh = _hip.conv_desc(f64, (2, 3, 8, 8), (4, 3, 3, 3), (8, 8), (1, 1), (1, 1), (1, 1))
    assert fresh is not c  # the builders themselves always build
