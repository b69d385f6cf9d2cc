"""The drop-in path on the GPU: conv_nd / max_pool called like the reference's
functions, gradients through Tensor.backward(), checked against the CPU oracle.
Bars: pooling bit-exact; convolution 1e-10 (float64) / 2e-4 (float32) in
max-abs error normalised by the reference's max-abs."""

import numpy as np
import pytest

import mygrad_amd as mg
from mygrad_amd import _device, _graph
from mygrad_amd.nnet import conv_nd, max_pool
from oracle import direct
from oracle import np_oracle as ora

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float64): 1e-10, np.dtype(np.float32): 2e-4}


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    if not mg.is_available():
        pytest.fail("libmygrad_hip.so / gfx950 device not available: the GPU tests need both")


def rel_err(got, want):
    scale = float(np.max(np.abs(want))) or 1.0
    return float(np.max(np.abs(np.asarray(got, np.float64) - np.asarray(want, np.float64)))) / scale


def test_reference_docstring_and_known_answers(kats):
    for case in kats["conv"]:
        x, w = mg.Tensor(np.array(case["x"], dtype=float)), mg.Tensor(np.array(case["w"], dtype=float))
        conf = dict(stride=tuple(case["stride"]), padding=tuple(case["padding"]), dilation=tuple(case["dilation"]))
        out = conv_nd(x, w, **conf)
        assert isinstance(out, mg.Tensor) and out.constant is False
        assert np.array_equal(out.data, np.array(case["out"], dtype=float)), case["source"]
        out.backward()
        if "dx_of_ones" in case:
            assert np.array_equal(x.grad, np.array(case["dx_of_ones"], dtype=float))
            assert np.array_equal(w.grad, np.array(case["dw_of_ones"], dtype=float))
        assert conv_nd(x, w, constant=True, **conf).constant is True
        x.clear_graph(), w.clear_graph()
    for case in kats["pool"]:
        x = mg.Tensor(np.array(case["x"]), dtype=case["dtype"])
        out = max_pool(x, tuple(case["pool"]), tuple(case["stride"]))
        assert np.array_equal(out.data, np.array(case["out"], dtype=x.dtype)), case["source"]
        if case["grad"] is None:
            out.clear_graph()
            continue
        if case["grad"] == "ones":
            out.backward()
        else:
            out.backward(np.arange(out.size).reshape(out.shape))
        assert x.grad.dtype == x.dtype
        assert np.array_equal(x.grad, np.array(case["dx"], dtype=float)), case["source"]
        assert max_pool(x, tuple(case["pool"]), tuple(case["stride"]), constant=True).constant is True
    assert _graph.held_count() == 0


@pytest.mark.parametrize("m", [1, 2, 3, 4])
def test_padding_only_image_gives_zero(m):
    rng = np.random.default_rng(m)
    pad = tuple(int(p) for p in rng.integers(1, 4, m))
    x = mg.Tensor(np.zeros((1, 1) + (0,) * m))
    w = rng.standard_normal((1, 1) + tuple(2 * p for p in pad))
    out = conv_nd(x, w, padding=pad, stride=1)
    assert out.shape == (1,) * (m + 2) and out.item() == 0.0
    out.backward()
    assert x.grad.shape == x.shape


def _drop_in_conv(seed, dtype, x_shape, w_shape, wscale, conf):
    rng = np.random.default_rng(seed)
    x = mg.Tensor(rng.standard_normal(x_shape).astype(dtype))
    w = mg.Tensor((rng.standard_normal(w_shape) * wscale).astype(dtype))
    out = conv_nd(x, w, **conf)
    g = rng.standard_normal(out.shape).astype(dtype)
    assert not x.data.flags.writeable and not out.data.flags.writeable
    out_data = out.data
    out.backward(g)
    assert x.data.flags.writeable and out_data.flags.writeable and _graph.held_count() == 0
    assert x.grad.dtype == dtype and w.grad.dtype == dtype and out.grad.dtype == dtype
    assert x.grad.shape == x.shape and w.grad.shape == w.shape
    assert not np.shares_memory(x.grad, g) and not np.shares_memory(w.grad, g)
    return x, w, g, out_data


def test_config1_through_backward():
    conf = dict(stride=1, padding=1, dilation=1)
    x, w, g, out = _drop_in_conv(1001, np.float64, (32, 3, 32, 32), (16, 3, 3, 3), 27 ** -0.5, conf)
    assert rel_err(out, ora.conv_forward(x.data, w.data, **conf)) <= 1e-10
    assert rel_err(x.grad, ora.conv_backward_x(g, x.shape, x.dtype, w.data, **conf)) <= 1e-10
    assert rel_err(w.grad, ora.conv_backward_w(g, x.data, w.shape, **conf)) <= 1e-10


def test_config3b_valid_through_backward():
    # (128,128,27,27): the neighbouring shape the reference accepts, same output (128,256,14,14)
    conf = dict(stride=2, padding=1, dilation=1)
    x, w, g, out = _drop_in_conv(1004, np.float32, (128, 128, 27, 27), (256, 128, 3, 3), (2 / 1152) ** 0.5, conf)
    assert out.shape == (128, 256, 14, 14)
    s, p, d = (2, 2), (1, 1), (1, 1)
    assert rel_err(out, direct.conv_forward(x.data, w.data, s, p, d)) <= 2e-4
    assert rel_err(x.grad, direct.conv_backward_x(g, x.shape, w.data, s, p, d)) <= 2e-4
    assert rel_err(w.grad, direct.conv_backward_w(g, x.data, w.shape, s, p, d)) <= 2e-4
    nb = 4
    assert rel_err(out[:nb], ora.conv_forward(x.data[:nb], w.data, **conf)) <= 2e-4
    assert rel_err(x.grad[:nb], ora.conv_backward_x(g[:nb], x.data[:nb].shape, x.dtype, w.data, **conf)) <= 2e-4


def test_config4_valid_through_backward():
    # (16,32,127,128) with padding (4,4): exact placements, output (16,32,64,128)
    conf = dict(stride=(2, 1), padding=(4, 4), dilation=(2, 2))
    x, w, g, out = _drop_in_conv(1005, np.float64, (16, 32, 127, 128), (32, 32, 5, 5), 800 ** -0.5, conf)
    assert out.shape == (16, 32, 64, 128)
    s, p, d = (2, 1), (4, 4), (2, 2)
    assert rel_err(out, direct.conv_forward(x.data, w.data, s, p, d)) <= 1e-10
    assert rel_err(x.grad, direct.conv_backward_x(g, x.shape, w.data, s, p, d)) <= 1e-10
    assert rel_err(w.grad, direct.conv_backward_w(g, x.data, w.shape, s, p, d)) <= 1e-10
    assert rel_err(out[:1], ora.conv_forward(x.data[:1], w.data, **conf)) <= 1e-10


@pytest.mark.parametrize("ties", [False, True])
def test_config2_valid_through_backward(ties):
    rng = np.random.default_rng(1002)
    shape = (64, 64, 55, 55)
    xv = rng.integers(0, 8, shape).astype(np.float64) if ties else rng.standard_normal(shape)
    x = mg.Tensor(xv)
    out = max_pool(x, (3, 3), 2)
    assert out.shape == (64, 64, 27, 27)
    g = rng.standard_normal(out.shape)
    out_data = out.data
    out.backward(g)
    want_out, want_dx = direct.pool(xv, g, (3, 3), (2, 2))
    assert np.array_equal(out_data.view(np.uint64), want_out.view(np.uint64))
    assert np.array_equal(x.grad.view(np.uint64), want_dx.view(np.uint64))
    sl = slice(0, 3)
    assert np.array_equal(out_data[sl], ora.pool_forward(xv[sl], (3, 3), 2))
    assert np.array_equal(x.grad[sl].view(np.uint64), ora.pool_backward(xv[sl], g[sl], (3, 3), 2).view(np.uint64))


def test_config5_chain_keeps_activations_on_the_device():
    rng = np.random.default_rng(1006)
    dtype = np.float32
    x = mg.Tensor(rng.standard_normal((8, 16, 32, 64, 64)).astype(dtype))
    w = mg.Tensor((rng.standard_normal((32, 16, 3, 3, 3)) * (2 / 432) ** 0.5).astype(dtype))
    g = rng.standard_normal((8, 32, 16, 32, 32)).astype(dtype)
    before = dict(_device.stats)
    y = conv_nd(x, w, stride=1, padding=1)
    z = max_pool(y, (2, 2, 2), 2)
    y_data, z_data = y.data, z.data
    z.backward(g)
    uploads = _device.stats["uploads"] - before["uploads"]
    assert uploads == 3, uploads  # x, w and the seed gradient; nothing is uploaded twice
    assert _device.stats["mirror_hits"] - before["mirror_hits"] >= 5

    s = p = d = (1, 1, 1)
    assert rel_err(y_data, direct.conv_forward(x.data, w.data, s, p, d)) <= 2e-4
    want_z, want_dy = direct.pool(y_data, g, (2, 2, 2), (2, 2, 2))
    assert np.array_equal(z_data, want_z)
    assert np.array_equal(y.grad.view(np.uint32), want_dy.astype(dtype).view(np.uint32))
    assert rel_err(x.grad, direct.conv_backward_x(y.grad, x.shape, w.data, s, p, d)) <= 2e-4
    assert rel_err(w.grad, direct.conv_backward_w(y.grad, x.data, w.shape, s, p, d)) <= 2e-4
    assert _graph.held_count() == 0


def test_max_pool_keeps_each_windows_argmax_only_while_x_is_guarded():
    """The forward pass records where every window's maximum sits and the backward pass
    routes by that record; with the memory guard off x may change in between, and then
    the maxima are found again from the x of that moment, as the reference does."""
    rng = np.random.default_rng(77)
    xv = rng.integers(0, 4, (3, 2, 9, 11)).astype(np.float32)  # ties everywhere
    g = rng.standard_normal((3, 2, 4, 5)).astype(np.float32)
    x = mg.Tensor(xv.copy())
    out = max_pool(x, (3, 3), 2)
    assert out.creator._argmax is not None and _device.is_locked(x.data)
    out.backward(g)
    want = ora.pool_backward(xv, g, (3, 3), 2).astype(np.float32)
    assert np.array_equal(x.grad.view(np.uint32), want.view(np.uint32))

    big = mg.Tensor(rng.integers(0, 30, (2, 20, 20)).astype(np.float64))  # 272 positions per window
    out = max_pool(big, (17, 16), 1)
    assert out.creator._argmax is None
    out.backward()
    assert np.array_equal(big.grad, ora.pool_backward(big.data, np.ones((2, 4, 5)), (17, 16), 1))

    with mg.mem_guard_off:
        x = mg.Tensor(xv.copy())
        out = max_pool(x, (3, 3), 2)
        assert not _device.is_locked(x.data)
        x.data[...] = x.data[..., ::-1].copy()  # allowed without the guard
        out.backward(g)
        want = ora.pool_backward(xv[..., ::-1], g, (3, 3), 2).astype(np.float32)
        assert np.array_equal(x.grad.view(np.uint32), want.view(np.uint32))
    assert _graph.held_count() == 0


def test_mirror_is_dropped_when_host_data_may_change():
    rng = np.random.default_rng(9)
    x = mg.Tensor(rng.standard_normal((2, 3, 8, 8)))
    w = mg.Tensor(rng.standard_normal((4, 3, 3, 3)))
    conv_nd(x, w, stride=1).backward()
    w.data[...] *= 2.0  # an optimiser step on the host between two graphs
    out = conv_nd(x, w, stride=1)
    assert rel_err(out.data, ora.conv_forward(x.data, w.data, stride=1)) <= 1e-10
    out.clear_graph()


def test_operand_variety():
    rng = np.random.default_rng(10)
    x64 = rng.standard_normal((2, 3, 9, 9))
    w32 = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    # mixed precision promotes like NumPy; gradients come back in each operand's dtype
    x, w = mg.Tensor(x64), mg.Tensor(w32)
    out = conv_nd(x, w, stride=2)
    assert out.dtype == np.float64
    out.backward()
    assert x.grad.dtype == np.float64 and w.grad.dtype == np.float32
    assert rel_err(out.data, ora.conv_forward(x64, w32, stride=2)) <= 1e-10
    # non-contiguous operands and integer (constant) data
    xt = mg.Tensor(np.asfortranarray(x64))
    xi = mg.Tensor(rng.integers(-3, 4, (2, 3, 9, 9)))
    wt = mg.Tensor(w32.astype(np.float64))
    assert rel_err(conv_nd(xt, wt, stride=1).data, ora.conv_forward(x64, wt.data, stride=1)) <= 1e-10
    out = conv_nd(xi, wt, stride=1, dilation=2)
    assert out.dtype == np.float64
    assert rel_err(out.data, ora.conv_forward(xi.data, wt.data, stride=1, dilation=2)) <= 1e-10
    out.backward()
    assert xi.grad is None and wt.grad is not None
    # only one non-constant input: only that gradient is computed
    xc = mg.Tensor(x64, constant=True)
    out = conv_nd(xc, wt, stride=1)
    out.backward()
    assert xc.grad is None
    assert rel_err(wt.grad, ora.conv_backward_w(np.ones(out.shape), x64, wt.shape, stride=1)) <= 1e-10
    # pooling over all axes of a 2-D tensor (no leading axes) and over a non-contiguous one
    p = mg.Tensor(np.asfortranarray(rng.integers(0, 5, (6, 8)).astype(np.float64)))
    out = max_pool(p, (2, 2), (2, 2))
    assert np.array_equal(out.data, ora.pool_forward(p.data, (2, 2), 2))
    out.backward()
    assert np.array_equal(p.grad, ora.pool_backward(p.data, np.ones(out.shape), (2, 2), 2))
    assert _graph.held_count() == 0


def test_a_layer_called_again_reuses_its_checks_but_not_for_other_settings():
    """ConvND keeps what its argument checks derived for a (shapes, settings) pair and the shared
    descriptor of the layer: a second call gives the same result, other settings on the same shapes
    get their own entry, and settings that the checks reject are rejected every time."""
    rng = np.random.default_rng(77)
    x, w = rng.standard_normal((2, 3, 9, 9)), rng.standard_normal((4, 3, 3, 3))
    first = conv_nd(x, w, stride=1, padding=1, constant=True).data
    again = conv_nd(x, w, stride=1, padding=1, constant=True).data
    assert np.array_equal(first, again)
    assert rel_err(first, direct.conv_forward(x, w, (1, 1), (1, 1), (1, 1))) < TOL[np.dtype(np.float64)]
    for conf in (dict(stride=2, padding=0), dict(stride=(1, 1), padding=(0, 1)), dict(stride=1, padding=1, dilation=2),
                 dict(stride=[1, 1], padding=np.array([1, 1]))):
        stride, padding, dilation = (np.broadcast_to(np.asarray(conf.get(k, d)), (2,)) for k, d in
                                     (("stride", 1), ("padding", 0), ("dilation", 1)))
        if any((n + 2 * p - ((t - 1) * d + 1)) % s for n, t, s, p, d in zip((9, 9), (3, 3), stride, padding, dilation)):
            with pytest.raises(ValueError):
                conv_nd(x, w, **conf)
            continue
        for _ in range(2):
            got = conv_nd(x, w, constant=True, **conf).data
            want = direct.conv_forward(x, w, tuple(int(v) for v in stride), tuple(int(v) for v in padding),
                                       tuple(int(v) for v in dilation))
            assert got.shape == want.shape and rel_err(got, want) < TOL[np.dtype(np.float64)]
    for _ in range(2):  # rejected before and after good calls with the same shapes
        with pytest.raises(AssertionError):
            conv_nd(x, w, stride=0, padding=1)
        with pytest.raises(AssertionError):
            conv_nd(x, w, stride=1, padding=(1, 1, 1))
        with pytest.raises(ValueError):
            conv_nd(x, w, stride=3, padding=1)
    out = conv_nd(mg.Tensor(x), mg.Tensor(w), stride=1, padding=1)
    assert not out.creator.stride.flags.writeable  # the arrays are shared between the operations of a layer


def test_integer_operands_give_the_integer_result():
    """All-integer operands are constants; the reference multiplies them in integer arithmetic
    (np.tensordot, conv.py:96-99) and takes maxima of integers (pooling.py:93).  Here they run in
    float64, exactly, and come back in NumPy's result type."""
    rng = np.random.default_rng(14)
    xi = rng.integers(-1000, 1000, (3, 4, 11, 12))
    wi = rng.integers(-50, 50, (5, 4, 3, 2)).astype(np.int32)
    out = conv_nd(xi, wi, stride=(2, 1), padding=(1, 0), dilation=(1, 2))
    want = ora.conv_forward(xi, wi, stride=(2, 1), padding=(1, 0), dilation=(1, 2))
    assert out.dtype == want.dtype == np.int64 and out.constant and np.array_equal(out.data, want)
    pooled = max_pool(mg.Tensor(xi.astype(np.int16)), (3, 2), (2, 2))
    assert pooled.dtype == np.int16 and np.array_equal(pooled.data, ora.pool_forward(xi.astype(np.int16), (3, 2), (2, 2)))
    big = np.array([[2**53 - 1, -(2**53) + 1, 0, 5]])
    assert np.array_equal(max_pool(big, (2,), 2).data, [[2**53 - 1, 5]])
    del out, pooled  # the results hold their operands read-only for as long as they live
    assert _graph.held_count() == 0


def test_tensor_feeding_two_pools_accumulates_like_the_reference():
    # second contribution is added to an existing float32 gradient: the reference adds
    # the unrounded float64 dx (pooling.py:147, operation_base.py:227-228)
    rng = np.random.default_rng(12)
    xv = rng.integers(0, 3, (3, 9, 9)).astype(np.float32)
    x = mg.Tensor(xv)

    class Twice(mg.Operation):
        def __call__(self, a, b):
            self.variables = (a, b)
            return a.data + b.data

        def backward_var(self, grad, index, **kwargs):
            return grad * np.float32(1.0 if index == 0 else 3.0)

    a = max_pool(x, (3, 3), 1)
    b = max_pool(x, (3, 3), 1)
    out = mg.execute_op(Twice, a, b)
    g = (rng.standard_normal(out.shape) * 1e3).astype(np.float32)
    out.backward(g)
    first = ora.pool_backward(xv, g * np.float32(1.0), (3, 3), 1)
    second = ora.pool_backward(xv, g * np.float32(3.0), (3, 3), 1)
    # backward visits `b` (the later consumer in topological order) or `a` first;
    # either way: float32(first-visited), then += the other in float64
    want_ab = first.astype(np.float32)
    want_ab += second
    want_ba = second.astype(np.float32)
    want_ba += first
    assert np.array_equal(x.grad, want_ab) or np.array_equal(x.grad, want_ba)


def test_config3a_through_backward():
    conf = dict(stride=1, padding=1, dilation=1)
    x, w, g, out = _drop_in_conv(1003, np.float32, (128, 64, 56, 56), (64, 64, 3, 3), (2 / 576) ** 0.5, conf)
    assert out.shape == (128, 64, 56, 56)
    s = p = d = (1, 1)
    assert rel_err(out, direct.conv_forward(x.data, w.data, s, p, d)) <= 2e-4
    assert rel_err(x.grad, direct.conv_backward_x(g, x.shape, w.data, s, p, d)) <= 2e-4
    assert rel_err(w.grad, direct.conv_backward_w(g, x.data, w.shape, s, p, d)) <= 2e-4
    nb = 2
    assert rel_err(out[:nb], ora.conv_forward(x.data[:nb], w.data, **conf)) <= 2e-4
    assert rel_err(x.grad[:nb], ora.conv_backward_x(g[:nb], x.data[:nb].shape, x.dtype, w.data, **conf)) <= 2e-4


def test_config5_chain_copies_back_only_what_is_read():
    """Nothing a kernel wrote crosses PCIe until somebody reads it: for the conv -> relu -> pool
    -> sum(. * g) chain the bytes copied device-to-host are those of the loss, x.grad and w.grad."""
    from mygrad_amd.nnet import relu

    rng = np.random.default_rng(1006)
    dtype = np.float32
    xv = rng.standard_normal((8, 16, 32, 64, 64)).astype(dtype)
    wv = (rng.standard_normal((32, 16, 3, 3, 3)) * (2 / 432) ** 0.5).astype(dtype)
    gv = rng.standard_normal((8, 32, 16, 32, 32)).astype(dtype)
    x, w, g = mg.Tensor(xv), mg.Tensor(wv), mg.Tensor(gv, constant=True)
    before = dict(_device.stats)
    y = conv_nd(x, w, stride=1, padding=1)
    z = max_pool(relu(y), (2, 2, 2), 2)
    loss = mg.sum(z * g)
    assert y.on_device and z.on_device and loss.on_device
    loss.backward()
    assert _device.stats["d2h_bytes"] == before["d2h_bytes"]  # nothing has been read yet
    assert _device.stats["uploads"] - before["uploads"] == 3  # x, w, g
    loss_value = loss.item()
    dx, dw = x.grad, w.grad
    assert _device.stats["d2h_bytes"] - before["d2h_bytes"] == dx.nbytes + dw.nbytes + 4
    assert y.on_device and z.on_device and y.grad is not None
    assert dx.flags.writeable and dw.flags.writeable and dx.dtype == dtype and dw.dtype == dtype

    # the same numbers as the oracle's, step by step (reading y, z now copies them back)
    s = p = d = (1, 1, 1)
    y_data = y.data
    assert rel_err(y_data, direct.conv_forward(xv, wv, s, p, d)) <= 2e-4
    r = ora.relu_forward(y_data)
    want_z, dr = direct.pool(r, gv, (2, 2, 2), (2, 2, 2))
    assert np.array_equal(z.data, want_z)
    assert abs(loss_value - float(np.sum(want_z.astype(np.float64) * gv))) <= 1e-6 * float(np.sum(np.abs(want_z * gv)))
    dy = ora.relu_backward(y_data, dr.astype(dtype))
    assert np.array_equal(y.grad.view(np.uint32), dy.view(np.uint32))
    assert rel_err(dx, direct.conv_backward_x(dy, xv.shape, wv, s, p, d)) <= 2e-4
    assert rel_err(dw, direct.conv_backward_w(dy, xv, wv.shape, s, p, d)) <= 2e-4
    assert _graph.held_count() == 0


def test_result_read_while_the_graph_is_alive_is_held_read_only():
    rng = np.random.default_rng(21)
    x = mg.Tensor(rng.standard_normal((2, 3, 8, 8)))
    w = mg.Tensor(rng.standard_normal((4, 3, 3, 3)))
    y = conv_nd(x, w, stride=1)
    z = max_pool(y, (2, 2), 2)
    assert y.on_device and z.on_device
    y_data = y.data  # read after two operations took hold of it: both must release it
    assert not y.on_device and not y_data.flags.writeable and y.data is y_data
    with pytest.raises(ValueError):
        y_data[...] = 0.0
    uploads = _device.stats["uploads"]
    z.backward()
    assert _device.stats["uploads"] == uploads  # the host copy of y did not have to go back up
    assert y_data.flags.writeable and _graph.held_count() == 0
    want_dy = ora.pool_backward(y_data, np.ones(z.shape), (2, 2), 2)
    assert np.array_equal(y.grad, want_dy)
    assert rel_err(x.grad, ora.conv_backward_x(want_dy, x.shape, x.dtype, w.data, stride=1)) <= 1e-10
    # a result read after its graph is gone is an ordinary writeable array
    y2 = conv_nd(x, w, stride=1)
    y2.clear_graph()
    assert y2.data.flags.writeable


def test_unguarded_result_edited_on_the_host_is_uploaded_again():
    """Under no_autodiff (or without the memory guard) a result is handed out writeable; a later
    operation must see the host's edits, not a device copy kept from before them."""
    rng = np.random.default_rng(22)
    x = rng.standard_normal((2, 3, 8, 8))
    w = rng.standard_normal((4, 3, 3, 3))
    for switch in (mg.no_autodiff, mg.mem_guard_off):
        with switch:
            y = conv_nd(x, w, stride=1)
        assert y.data.flags.writeable
        y.data[...] = rng.standard_normal(y.shape)
        z = max_pool(y, (2, 2), 2)
        assert np.array_equal(z.data, ora.pool_forward(y.data, (2, 2), 2))
        z.clear_graph()
    # the eager contract (an operation called directly returns a host array): same rule
    from mygrad_amd.nnet.layers.conv import ConvND

    out = ConvND()(mg.Tensor(x), mg.Tensor(w), stride=1)
    assert isinstance(out, np.ndarray) and out.flags.writeable
    out[...] = 1.0
    z = max_pool(out, (2, 2), 2)
    assert np.array_equal(z.data, np.ones(z.shape))
    z.clear_graph()
    assert _graph.held_count() == 0


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_gradients_of_a_tensor_used_twice_are_added_on_the_device(dtype):
    from mygrad_amd.nnet import relu

    rng = np.random.default_rng(23)
    xv = rng.standard_normal((3, 4, 9, 9)).astype(dtype)
    wv = rng.standard_normal((5, 4, 3, 3)).astype(dtype)
    gv = rng.standard_normal((3, 5, 7, 7)).astype(dtype)
    x, w = mg.Tensor(xv), mg.Tensor(wv)
    a = conv_nd(x, w, stride=1)
    b = conv_nd(x, w, stride=1)  # x and w feed two operations: their gradients are sums of two terms
    out = relu(a) * b
    before = _device.stats["d2h_bytes"]
    out.backward(gv)
    assert _device.stats["d2h_bytes"] == before
    ya = ora.conv_forward(xv, wv, stride=1)
    da = ora.relu_backward(ya, (gv * ya).astype(dtype))
    db = (gv * ora.relu_forward(ya)).astype(dtype)
    want_dx = ora.conv_backward_x(da, xv.shape, xv.dtype, wv, stride=1) + ora.conv_backward_x(db, xv.shape, xv.dtype, wv, stride=1)
    want_dw = ora.conv_backward_w(da, xv, wv.shape, stride=1) + ora.conv_backward_w(db, xv, wv.shape, stride=1)
    tol = TOL[np.dtype(dtype)]
    assert x.grad.dtype == dtype and rel_err(x.grad, want_dx) <= tol
    assert rel_err(w.grad, want_dw) <= tol
    assert _graph.held_count() == 0


def test_device_tensor_is_uploaded_once_and_seeds_backward():
    rng = np.random.default_rng(24)
    xv = rng.standard_normal((2, 3, 10, 10)).astype(np.float32)
    wv = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    gv = rng.standard_normal((2, 4, 8, 8)).astype(np.float32)
    before = dict(_device.stats)
    x, w, g = mg.device_tensor(xv), mg.device_tensor(wv), mg.device_tensor(gv, constant=True)
    assert x.on_device and x.shape == xv.shape and x.dtype == np.float32 and not x.constant
    for _ in range(3):  # three graphs over the same tensors: nothing goes up or comes down again
        out = conv_nd(x, w, stride=1)
        out.backward(g)
    assert _device.stats["uploads"] - before["uploads"] == 3
    assert _device.stats["d2h_bytes"] == before["d2h_bytes"]
    assert rel_err(x.grad, ora.conv_backward_x(gv, xv.shape, xv.dtype, wv, stride=1)) <= 2e-4
    assert rel_err(w.grad, ora.conv_backward_w(gv, xv, wv.shape, stride=1)) <= 2e-4
    assert np.array_equal(x.data, xv) and x.data.flags.writeable
    with pytest.raises(TypeError):
        mg.device_tensor(np.arange(4))
    assert _graph.held_count() == 0


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_four_and_five_convolved_axes(dtype):
    """More convolved axes than the kernels take: the leading ones are taken apart on the host
    into convolutions over the last three (the reference takes any number, conv.py:23-29)."""
    from oracle import brute

    rng = np.random.default_rng(31)
    tol = TOL[np.dtype(dtype)]
    cases = [
        # x shape, w shape, stride, padding, dilation
        ((2, 3, 5, 7, 5, 7), (4, 3, 2, 3, 2, 3), (1, 2, 1, 2), (1, 0, 1, 1), (2, 1, 1, 1)),
        ((1, 16, 4, 6, 6, 8), (16, 16, 3, 1, 3, 3), (1, 1, 1, 1), (1, 0, 1, 1), (1, 1, 1, 1)),
        ((2, 2, 3, 4, 3, 4, 5), (3, 2, 2, 2, 1, 2, 2), (1, 1, 1, 1, 1), (0, 1, 0, 0, 1), (1, 1, 1, 1, 1)),
    ]
    for x_shape, w_shape, s, p, d in cases:
        xv = rng.standard_normal(x_shape).astype(dtype)
        wv = (rng.standard_normal(w_shape) / np.sqrt(np.prod(w_shape[1:]))).astype(dtype)
        x, w = mg.Tensor(xv), mg.Tensor(wv)
        out = conv_nd(x, w, stride=s, padding=p, dilation=d)
        want = ora.conv_forward(xv, wv, stride=s, padding=p, dilation=d)
        assert out.shape == want.shape and out.dtype == dtype
        g = rng.standard_normal(out.shape).astype(dtype)
        out_data = out.data
        out.backward(g)
        assert rel_err(out_data, want) <= tol
        assert rel_err(x.grad, ora.conv_backward_x(g, xv.shape, xv.dtype, wv, stride=s, padding=p, dilation=d)) <= tol
        assert rel_err(w.grad, ora.conv_backward_w(g, xv, wv.shape, stride=s, padding=p, dilation=d)) <= tol
        if xv.size * wv.size // wv.shape[1] < 3_000_000:  # the definition itself, in loops
            assert rel_err(out_data, brute.conv_forward(xv, wv, s, p, d)) <= tol
    assert _graph.held_count() == 0


MANY_AXES_POOLS = [
    # x shape, pool, stride: four to seven axes that are really pooled, windows that overlap along
    # leading and trailing axes, un-pooled axes in front, a last-three window of more than 256
    # positions (no argmax bytes for that stage)
    ((4, 4, 4, 4), (2, 2, 2, 2), (2, 2, 2, 2)),
    ((2, 5, 6, 7, 8), (3, 2, 3, 2), (1, 2, 2, 3)),
    ((3, 4, 5, 4, 6, 5), (2, 1, 2, 3, 2), (1, 2, 1, 1, 3)),
    ((2, 3, 2, 3, 4, 5, 4), (2, 2, 3, 2, 2, 2), (1, 1, 1, 2, 3, 2)),
    ((2, 2, 3, 2, 2, 3, 4, 3), (2, 2, 2, 2, 2, 2, 2), (1, 1, 1, 1, 1, 2, 1)),
    ((3, 4, 9, 10, 8), (2, 7, 8, 5), (1, 2, 2, 3)),
]


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("case", range(len(MANY_AXES_POOLS)))
def test_pooling_over_more_axes_than_the_kernels_take(case, dtype):
    """More than three pooled axes run as stages of three (mygrad/nnet/layers/pooling.py:21-25 takes
    any number); values and the first-in-row-major-order routing of ties must come out as from
    the one-pass definition.  Small integers: every sum is exact, so dx is compared bit for bit."""
    x_shape, pool, stride = MANY_AXES_POOLS[case]
    rng = np.random.default_rng(4000 + case)
    xv = rng.integers(0, 3, x_shape).astype(dtype)  # ties in nearly every window
    x = mg.Tensor(xv)
    out = max_pool(x, pool, stride)
    want = ora.pool_forward(xv, pool, stride, validate=False)
    assert out.shape == want.shape and np.array_equal(out.data, want)
    g = rng.integers(-3, 4, out.shape).astype(dtype)
    out.backward(g)
    want_dx = ora.pool_backward(xv, g, pool, stride)
    assert x.grad.dtype == dtype and np.array_equal(x.grad, want_dx.astype(dtype))
    # a second gradient added to the first (the float64 route), with real-valued gradients:
    # x feeds two poolings whose outputs are multiplied, so each sends g1 * (the other's output) back
    x2 = mg.Tensor(xv)
    g1 = rng.standard_normal(out.shape).astype(dtype)
    a, b = max_pool(x2, pool, stride), max_pool(x2, pool, stride)
    mg.sum(a * b * g1).backward()
    both = 2 * ora.pool_backward(xv, (g1 * want).astype(dtype), pool, stride)
    assert rel_err(x2.grad, both) <= (1e-6 if dtype == np.float32 else 1e-14)
    # with the memory guard off x may change after the forward pass: every stage finds its maxima again
    with mg.mem_guard_off:
        x3 = mg.Tensor(xv.copy())
        out3 = max_pool(x3, pool, stride)
        x3.data[...] = xv[::-1]
        out3.backward(g)
    assert np.array_equal(x3.grad, ora.pool_backward(np.ascontiguousarray(xv[::-1]), g, pool, stride).astype(dtype))
    assert _graph.held_count() == 0


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("x_shape,pool,stride", [
    ((2, 7, 6, 7, 8), (3, 2, 3, 2), (1, 2, 2, 3)),          # four pooled axes, windows that overlap along three of them
    ((3, 5, 6, 5, 7, 9), (2, 3, 2, 3, 3), (1, 1, 1, 2, 2)),  # five
    ((6, 5, 5, 5), (3, 3, 3, 3), (1, 1, 1, 1)),              # every element under up to 81 windows, no leading axes
    # six and seven pooled axes: three stages, three records
    ((2, 4, 5, 4, 5, 6, 5), (2, 3, 2, 3, 2, 3), (1, 1, 2, 1, 2, 1)),
    ((3, 4, 3, 4, 3, 5, 4), (2, 2, 2, 2, 2, 3, 2), (1, 1, 1, 2, 1, 1, 2)),
])
def test_pooling_over_four_and_five_axes_adds_in_the_reference_order(x_shape, pool, stride, dtype):
    """Real-valued gradients of very different magnitudes: the sum an element receives depends on
    the order of its terms, and must be np.add.at's (pooling.py:147-148) bit for bit -- also for a
    float32 x, whose sums the reference carries in float64 and rounds once.  (Four to seven pooled
    axes: two or three stages of the kernels' three axes.)"""
    rng = np.random.default_rng(4100 + len(pool))
    xv = rng.integers(0, 3, x_shape).astype(dtype)  # ties: an element is the argmax of many windows
    out_shape = ora.pool_forward(xv, pool, stride).shape
    g = (rng.standard_normal(out_shape) * 10.0 ** rng.integers(-6, 6, out_shape)).astype(dtype)
    g[rng.random(out_shape) < 0.1] = -0.0
    x = mg.Tensor(xv)
    max_pool(x, pool, stride).backward(g)
    from mygrad_amd import _hip

    assert ("three" if len(pool) > 5 else "two") + " stages' argmax" in _hip.last_plan()
    want = ora.pool_backward(xv, g, pool, stride)  # float64
    kind = np.uint64 if dtype == np.float64 else np.uint32
    assert np.array_equal(x.grad.view(kind), want.astype(dtype).view(kind))
    # the float64 route (a gradient that is added to one the tensor already holds): x feeds two
    # poolings whose outputs are multiplied, so each sends g * (the other's output) back
    x2 = mg.Tensor(xv)
    a, b = max_pool(x2, pool, stride), max_pool(x2, pool, stride)
    mg.sum(a * b * mg.Tensor(g, constant=True)).backward()
    sent = (g * ora.pool_forward(xv, pool, stride)).astype(dtype)  # one rounding, like the device's multiply
    each = ora.pool_backward(xv, sent, pool, stride)  # float64
    assert np.array_equal(x2.grad.view(kind), (each.astype(dtype).astype(np.float64) + each).astype(dtype).view(kind))
    assert _graph.held_count() == 0


def test_window_with_zeros_of_both_signs_keeps_the_first_ones_sign():
    """np.max over a window that holds +0.0 and -0.0 returns either, depending on the order and the
    vector width (implementation-defined); here the first of the equal maxima wins, as np.argmax
    picks it, and the gradient goes to that element."""
    for first, second in ((0.0, -0.0), (-0.0, 0.0)):
        x = mg.Tensor(np.array([[first, second, -1.0, second]]))
        out = max_pool(x, (4,), 4)
        assert np.signbit(out.data[0, 0]) == np.signbit(first)
        out.backward(np.array([[5.0]]))
        assert np.array_equal(x.grad, [[5.0, 0.0, 0.0, 0.0]])


def test_pooling_over_four_axes_with_a_leading_window_of_one():
    rng = np.random.default_rng(32)
    xv = rng.integers(0, 4, (2, 3, 5, 6, 8)).astype(np.float64)
    x = mg.Tensor(xv)
    out = max_pool(x, (1, 1, 2, 3, 2), (1, 1, 1, 3, 2))  # five pooled axes, two of them with a window of one element
    want = ora.pool_forward(xv, (1, 1, 2, 3, 2), (1, 1, 1, 3, 2), validate=False)
    assert np.array_equal(out.data, want)
    g = rng.standard_normal(out.shape)
    out.backward(g)
    assert np.array_equal(x.grad.view(np.uint64), ora.pool_backward(xv, g, (1, 1, 2, 3, 2), (1, 1, 1, 3, 2)).view(np.uint64))
    assert _graph.held_count() == 0


def _ulp16(a):
    return np.spacing(np.abs(np.asarray(a, dtype=np.float16))).astype(np.float64)


def test_casts_to_and_from_float16_round_like_numpy():
    """float16 is a storage type of the library: ``mg_cast`` rounds to nearest even in one step
    (a float64 just above a float16 tie must not be rounded to float32 first), keeps signed zeros,
    infinities, NaNs and subnormals, and ``mg_accumulate`` forms ``a += b`` in the wider type."""
    rng = np.random.default_rng(77)
    tie = 1.0 + 2.0**-11  # halfway between two float16 values
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 65504.0, 65519.9, 65520.0, -65520.0, 1e-8, 5.96e-8, 2.98e-8,
                        2.9803e-8, 6.1e-5, tie, tie + 2.0**-40, tie - 2.0**-40, -(tie + 2.0**-40), 3 * 2.0**-11 + 1, 2049.0, 2051.0], dtype=np.float64)
    values = np.concatenate([special, rng.standard_normal(5000) * 10.0 ** rng.integers(-9, 5, 5000)])
    for wide in (np.float64, np.float32):
        src = values.astype(wide)
        buf = _device.DeviceBuffer(max(src.nbytes, 16))
        buf.upload(src)
        with np.errstate(over="ignore"):
            want = src.astype(np.float16)
        got = _device.DeviceArray(buf, src.shape, wide).astype(np.float16)
        assert got.dtype == np.float16
        assert np.array_equal(got.host().view(np.uint16), want.view(np.uint16))
        back = got.astype(wide).host()
        assert np.array_equal(back.view(np.uint64 if wide == np.float64 else np.uint32), want.astype(wide).view(np.uint64 if wide == np.float64 else np.uint32))
    # a += b with a in float16: the sum is formed in the wider type and rounded once
    a16 = (rng.standard_normal(1000) * 8).astype(np.float16)
    for inc_dtype in (np.float16, np.float32, np.float64):
        inc = (rng.standard_normal(1000) * 8).astype(inc_dtype)
        abuf, ibuf = _device.DeviceBuffer(a16.nbytes), _device.DeviceBuffer(inc.nbytes)
        abuf.upload(a16)
        ibuf.upload(inc)
        acc = _device.DeviceArray(abuf, a16.shape, np.float16)
        acc.add_into(_device.DeviceArray(ibuf, inc.shape, inc_dtype))
        want = a16.copy()
        want += inc.astype(want.dtype, copy=False) if inc_dtype == np.float16 else inc  # NumPy: same-kind cast of the sum
        assert np.array_equal(acc.host().view(np.uint16), want.view(np.uint16)), inc_dtype


def test_float16_operands_are_widened_and_rounded_once():
    """float16 tensors (reference: any float dtype, conv.py:20-21; NumPy multiplies float16 arrays
    with float32 sums rounded to float16 at the end).  Here the operands are widened to float32,
    the float32 kernels run and the result is rounded once: within one float16 unit in the last
    place of the reference's value everywhere (the sums run in another order), and within half a
    unit (+ the float32 sum's own error) of the exact result, which the reference's dx -- rounded
    after every window it adds -- is not."""
    rng = np.random.default_rng(78)
    x16 = rng.standard_normal((4, 6, 12, 12)).astype(np.float16)
    w16 = (rng.standard_normal((8, 6, 3, 3)) / 7).astype(np.float16)
    x, w = mg.Tensor(x16), mg.Tensor(w16)
    out = conv_nd(x, w, stride=1, padding=1)
    assert out.dtype == np.float16 and out.shape == (4, 8, 12, 12)
    want = ora.conv_forward(x16, w16, stride=1, padding=1)
    assert want.dtype == np.float16
    got = out.data
    assert np.mean(got == want) > 0.98
    # the exact result, and what a float32 sum of these terms may be off by (1e-6 of the sum of
    # their magnitudes: 54 to 576 terms of relative error 6e-8 each)
    x64, w64 = x16.astype(np.float64), w16.astype(np.float64)
    exact = ora.conv_forward(x64, w64, stride=1, padding=1)
    slack = 1e-6 * ora.conv_forward(np.abs(x64), np.abs(w64), stride=1, padding=1)
    assert np.all(np.abs(got.astype(np.float64) - exact) <= 0.5 * _ulp16(exact) + slack)
    assert np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= _ulp16(want) + 2 * slack)

    g16 = rng.standard_normal(out.shape).astype(np.float16)
    out.backward(g16)
    assert x.grad.dtype == np.float16 and w.grad.dtype == np.float16
    g64 = g16.astype(np.float64)
    dx_exact = ora.conv_backward_x(g64, x16.shape, np.float64, w64, stride=1, padding=1)
    dw_exact = ora.conv_backward_w(g64, x64, w16.shape, stride=1, padding=1)
    dx_slack = 1e-6 * ora.conv_backward_x(np.abs(g64), x16.shape, np.float64, np.abs(w64), stride=1, padding=1)
    dw_slack = 1e-6 * ora.conv_backward_w(np.abs(g64), np.abs(x64), w16.shape, stride=1, padding=1)
    assert np.all(np.abs(x.grad.astype(np.float64) - dx_exact) <= 0.5 * _ulp16(dx_exact) + dx_slack)
    assert np.all(np.abs(w.grad.astype(np.float64) - dw_exact) <= 0.5 * _ulp16(dw_exact) + dw_slack)
    # against the reference's own arithmetic: dw has one rounding there too, dx nine more
    dw_ref = ora.conv_backward_w(g16, x16, w16.shape, stride=1, padding=1)
    assert np.all(np.abs(w.grad.astype(np.float64) - dw_ref.astype(np.float64)) <= _ulp16(dw_ref) + 2 * dw_slack)
    dx_ref = ora.conv_backward_x(g16, x16.shape, np.float16, w16, stride=1, padding=1)
    assert rel_err(x.grad, dx_ref) <= 4e-3

    # float16 against float32 promotes to float32, as in NumPy
    out = conv_nd(mg.Tensor(x16), mg.Tensor(w16.astype(np.float32)), stride=1)
    assert out.dtype == np.float32
    assert rel_err(out.data, ora.conv_forward(x16.astype(np.float64), w16.astype(np.float64), stride=1)) <= 2e-4


def test_max_pool_of_float16_is_exact():
    """Pooling picks inputs and adds gradients in float64 (pooling.py:147), rounded to the tensor's
    type once: with float16 tensors both passes agree with the reference bit for bit, ties and
    overlapping windows included."""
    rng = np.random.default_rng(79)
    x16 = rng.integers(-4, 5, (3, 5, 13, 13)).astype(np.float16) / np.float16(4)  # many ties
    x16[0, 0, :4, :4] = rng.standard_normal((4, 4)).astype(np.float16) * 100
    g16 = (rng.standard_normal((3, 5, 6, 6)) * 3).astype(np.float16)
    x = mg.Tensor(x16)
    out = max_pool(x, (3, 3), 2)
    assert out.dtype == np.float16
    assert np.array_equal(out.data.view(np.uint16), ora.pool_forward(x16, (3, 3), 2).view(np.uint16))
    out.backward(g16)
    want = ora.pool_backward(x16, g16, (3, 3), 2).astype(np.float16)
    assert x.grad.dtype == np.float16
    assert np.array_equal(x.grad.view(np.uint16), want.view(np.uint16))


def test_float16_results_seed_backward_without_being_read():
    """backward() with no argument on a float16 result that is still on the device: the all-ones
    seed (tensor_base.py:1330-1334) is made on the device too, and the gradients are those of a
    seed of ones handed in from the host."""
    rng = np.random.default_rng(80)
    x16 = rng.standard_normal((2, 6, 9, 9)).astype(np.float16)
    w16 = (rng.standard_normal((4, 6, 3, 3)) / 7).astype(np.float16)
    for make in (lambda x, w: conv_nd(x, w, stride=2), lambda x, w: max_pool(conv_nd(x, w, stride=1), (3, 3), 2)):
        x, w = mg.Tensor(x16), mg.Tensor(w16)
        out = make(x, w)
        assert out.on_device and out.dtype == np.float16
        out.backward()
        x2, w2 = mg.Tensor(x16), mg.Tensor(w16)
        out2 = make(x2, w2)
        out2.backward(np.ones(out2.shape, dtype=np.float16))
        assert x.grad.dtype == np.float16 and w.grad.dtype == np.float16
        assert np.array_equal(x.grad.view(np.uint16), x2.grad.view(np.uint16))
        assert np.array_equal(w.grad.view(np.uint16), w2.grad.view(np.uint16))


def test_integer_result_on_the_device_meets_a_float_operand():
    """repeat() of an integer tensor leaves an integer array on the device; multiplying it by a
    float tensor converts it through the host, as NumPy would promote it."""
    a = np.arange(12, dtype=np.int64).reshape(3, 4)
    b = np.linspace(-1.0, 1.0, 24).reshape(3, 8)
    for dtype in (np.float64, np.float32):
        r = mg.repeat(mg.Tensor(a), 2, axis=1)
        assert r.dtype == np.int64
        f = mg.Tensor(b.astype(dtype))
        prod = r * f
        want = np.repeat(a, 2, axis=1) * b.astype(dtype)
        assert prod.dtype == want.dtype
        assert np.array_equal(prod.data, want)
        prod.backward()
        assert np.array_equal(f.grad, np.repeat(a, 2, axis=1).astype(dtype))


def test_weight_that_stays_on_the_device_keeps_no_dead_references():
    """A device tensor that is never read on the host (a weight in a training loop) remembers the
    operations that hold it read-only; the list must not grow with the number of steps."""
    rng = np.random.default_rng(81)
    w = mg.device_tensor(rng.standard_normal((8, 4, 3, 3)))
    x = mg.device_tensor(rng.standard_normal((2, 4, 8, 8)), constant=True)
    for _ in range(300):
        conv_nd(x, w, stride=1).backward()
    assert len(w._guards) <= 64 and len(x._guards) <= 64
    assert w.grad.shape == w.shape


def test_complex_operands_under_no_autodiff_carry_a_complex_step():
    """The reference's tests differentiate conv_nd numerically with a complex step through the
    operation itself (tests/nnet/layers/test_conv.py:291-300, tests/utils/numerical_gradient.py):
    complex128 operands under ``no_autodiff``.  Here they run as one real convolution of twice the
    channels and filters; the imaginary part of a step of 1e-20 comes back with full relative
    precision and gives the derivative the data gradient gives."""
    rng = np.random.default_rng(80)
    x = rng.standard_normal((2, 3, 9, 8))
    w = rng.standard_normal((4, 3, 3, 2))
    kwargs = dict(stride=(2, 1), padding=(1, 0), dilation=(1, 2))
    with mg.no_autodiff:
        z = conv_nd(x + 1j * rng.standard_normal(x.shape), w + 1j * rng.standard_normal(w.shape), **kwargs)
    assert z.dtype == np.complex128
    xc, wc = rng.standard_normal(x.shape) * 1j + x, rng.standard_normal(w.shape) * 1j + w
    with mg.no_autodiff:
        z = np.asarray(conv_nd(xc, wc, **kwargs).data)
    want = ora.conv_forward(xc, wc, **kwargs)
    assert rel_err(z.real, want.real) <= 1e-10 and rel_err(z.imag, want.imag) <= 1e-10

    # complex step in one element of x: d out / d x[e] for every output at once
    h = 1e-20
    e = (1, 2, 4, 3)
    step = x.astype(np.complex128)
    step[e] += 1j * h
    with mg.no_autodiff:
        slope = np.asarray(conv_nd(step, w.astype(np.complex128), **kwargs).data).imag / h
    g = rng.standard_normal(slope.shape)
    tx, tw = mg.Tensor(x), mg.Tensor(w)
    conv_nd(tx, tw, **kwargs).backward(g)
    assert abs(float(np.sum(slope * g)) - float(tx.grad[e])) <= 1e-10 * max(1.0, abs(float(tx.grad[e])))
    # a real operand against a complex one
    with mg.no_autodiff:
        z = np.asarray(conv_nd(x, wc, **kwargs).data)
    assert rel_err(z.imag, ora.conv_forward(x.astype(np.complex128), wc, **kwargs).imag) <= 1e-10
