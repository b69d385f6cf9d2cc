"""Parity of the matrix product (forward and both gradients) with the NumPy restatement of the
reference, through the C ABI and through ``Tensor.backward()``.

Bar: the convolution's -- maximum absolute error relative to the largest magnitude of the
expected array <= 1e-10 in float64, <= 2e-4 in float32 (the product runs on the convolution's
MFMA kernels; against a float64 evaluation for float32 inputs)."""

import numpy as np
import pytest

from oracle import np_oracle as ora

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 2e-4, np.dtype(np.float64): 1e-10}


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


# (batch, M, K, N): vectors, ragged sizes that are no multiple of any tile, one long reduction,
# tall / wide / batched operands
SIZES = [
    (1, 1, 1, 1),
    (1, 2, 2, 2),
    (1, 1, 7, 1),
    (1, 5, 3, 1),
    (1, 1, 3, 9),
    (1, 17, 33, 65),
    (3, 17, 33, 65),
    (1, 128, 128, 128),
    (1, 200, 1000, 72),
    (1, 64, 4099, 48),
    (2, 256, 96, 300),
    (1, 1024, 64, 16),
    (5, 16, 64, 1024),
    (1, 513, 257, 255),
    # large enough, with a reduction or a row count that is no multiple of 16: zero-padded operands
    (1, 520, 1000, 700),
    (2, 300, 330, 1100),
    (1, 512, 1000, 512),
    (1, 1001, 512, 512),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("batch, M, K, N", SIZES)
def test_product_and_gradients_match_the_oracle(abi, batch, M, K, N, dtype):
    dtype = np.dtype(dtype)
    rng = np.random.default_rng([batch, M, K, N])
    a = rng.standard_normal((M, K)).astype(dtype)
    x = rng.standard_normal((batch, K, N)).astype(dtype)
    g = rng.standard_normal((batch, M, N)).astype(dtype)
    wide = [v.astype(np.float64) for v in (a, x, g)]
    assert err(abi.matmul(a, x), ora.matmul_forward(wide[0], wide[1])) <= TOL[dtype]
    assert err(abi.matmul_da(g, x, M), ora.matmul_backward(wide[2], wide[0], wide[1], 0)) <= TOL[dtype]
    assert err(abi.matmul_dx(g, a), ora.matmul_backward(wide[2], wide[0], wide[1], 1)) <= TOL[dtype]


def test_results_repeat_exactly(abi):
    rng = np.random.default_rng(3)
    a = rng.standard_normal((96, 500)).astype(np.float32)
    x = rng.standard_normal((4, 500, 130)).astype(np.float32)
    g = rng.standard_normal((4, 96, 130)).astype(np.float32)
    for fn, args in ((abi.matmul, (a, x)), (abi.matmul_da, (g, x, 96)), (abi.matmul_dx, (g, a))):
        assert np.array_equal(fn(*args), fn(*args))


BATCHED = [(1, 1, 1, 1), (3, 16, 16, 16), (5, 17, 3, 33), (2, 1, 70, 1), (300, 8, 8, 8), (7, 64, 40, 48), (4, 33, 6, 2), (2, 5, 0, 4),
           (3, 100, 129, 50),
           # 32 x 32 results or more per pair: 64 x 64 tiles staged in LDS -- whole tiles, ragged edges in M, N
           # and K, several K chunks, row lengths that are and are not whole 16-byte pieces
           (9, 64, 64, 64), (3, 130, 70, 96), (2, 32, 200, 32), (5, 47, 33, 61), (2, 128, 64, 192)]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("batch, M, K, N", BATCHED)
def test_batched_product_with_and_without_transposed_operands(abi, batch, M, K, N, dtype):
    """mg_matmul_batched against float64 products of the same values, to the bar of the other
    matrix products (max abs error over the largest |entry|: 2e-4 float32, 1e-10 float64)."""
    dtype = np.dtype(dtype)
    rng = np.random.default_rng([batch, M, K, N])
    a, b = rng.standard_normal((batch, M, K)).astype(dtype), rng.standard_normal((batch, K, N)).astype(dtype)
    want = np.matmul(a.astype(np.float64), b.astype(np.float64))
    at, bt = np.ascontiguousarray(a.transpose(0, 2, 1)), np.ascontiguousarray(b.transpose(0, 2, 1))
    for ta, tb in ((False, False), (True, False), (False, True), (True, True)):
        got = abi.matmul_batched(at if ta else a, bt if tb else b, ta, tb)
        assert got.shape == want.shape and got.dtype == dtype
        assert err(got, want) <= TOL[dtype], (ta, tb)
    if K:  # a column and a row of the result must not see their neighbours: exact small integers
        ai, bi = np.round(a * 2), np.round(b * 2)
        assert np.array_equal(abi.matmul_batched(ai, bi), np.matmul(ai, bi))


def test_batched_product_bad_arguments(abi):
    from mygrad_amd import _device, _hip

    buf, lib = _device.DeviceBuffer(4096), _hip.lib()
    assert lib.mg_matmul_batched(0, 2, 4, 4, 4, 0, 0, buf.ptr, buf.ptr, buf.ptr) == _hip.MG_OK
    assert lib.mg_matmul_batched(2, 2, 4, 4, 4, 0, 0, buf.ptr, buf.ptr, buf.ptr) == _hip.MG_ERR_UNSUPPORTED
    assert lib.mg_matmul_batched(0, 2, -1, 4, 4, 0, 0, buf.ptr, buf.ptr, buf.ptr) == _hip.MG_ERR_BAD_ARG
    assert lib.mg_matmul_batched(0, 2, 4, 4, 4, 0, 0, None, buf.ptr, buf.ptr) == _hip.MG_ERR_BAD_ARG
    assert lib.mg_matmul_batched(0, 2, 4, 4, 4, 0, 0, buf.ptr, buf.ptr, None) == _hip.MG_ERR_BAD_ARG
    assert lib.mg_matmul_batched(0, 2, 1 << 24, 4, 4, 0, 0, buf.ptr, buf.ptr, buf.ptr) == _hip.MG_ERR_UNSUPPORTED
    assert lib.mg_matmul_batched(0, 0, 4, 4, 4, 0, 0, None, None, None) == _hip.MG_OK  # nothing to do


SHAPES = [
    ((3, 4), (4, 5)),
    ((4,), (4, 5)),
    ((3, 4), (4,)),
    ((4,), (4,)),
    ((2, 3, 4), (4, 5)),
    ((3, 4), (2, 4, 5)),
    ((2, 3, 4), (2, 4, 5)),
    ((4,), (2, 3, 4, 5)),
    ((2, 3, 4), (4,)),
    ((2, 2, 30, 40), (2, 2, 40, 50)),
    ((2, 800, 810), (2, 810, 790)),  # pairs large enough for a launch of the tiled kernels each
    ((60, 70), (70, 80)),
    # stacks that broadcast against each other
    ((2, 1, 3, 4), (2, 4, 5)),
    ((1, 3, 4), (2, 4, 5)),
    ((3, 1, 2, 6, 4), (2, 1, 4, 5)),
    ((2, 3, 4), (5, 1, 4, 3)),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("sa, sb", SHAPES)
def test_matmul_through_the_tensor_api(sa, sb, dtype):
    import mygrad_amd as mg

    dtype = np.dtype(dtype)
    rng = np.random.default_rng([len(sa), len(sb), int(np.prod(sa)), int(np.prod(sb))])
    a, b = mg.Tensor(rng.standard_normal(sa).astype(dtype)), mg.Tensor(rng.standard_normal(sb).astype(dtype))
    out = mg.matmul(a, b)
    wa, wb = a.data.astype(np.float64), b.data.astype(np.float64)
    want = ora.matmul_forward(wa, wb)
    assert out.shape == want.shape and out.dtype == dtype and err(out.data, want) <= TOL[dtype]
    g = rng.standard_normal(out.shape).astype(dtype)
    out.backward(g)
    assert a.grad.shape == sa and b.grad.shape == sb and a.grad.dtype == b.grad.dtype == dtype
    assert err(a.grad, ora.matmul_backward(g.astype(np.float64), wa, wb, 0)) <= TOL[dtype]
    assert err(b.grad, ora.matmul_backward(g.astype(np.float64), wa, wb, 1)) <= TOL[dtype]


def test_reference_vectors_operator_and_errors(kats):
    import mygrad_amd as mg
    for case in kats["matmul"]:
        if "a" not in case:
            out = mg.matmul(np.zeros(case["a_shape"]), np.zeros(case["b_shape"]))
            assert list(out.shape) == case["out_shape"]
            continue
        a, b = mg.Tensor(np.array(case["a"], dtype=float)), mg.Tensor(np.array(case["b"], dtype=float))
        out = a @ b
        assert np.array_equal(out.data, np.array(case["out"], dtype=float)), case["source"]
        out.backward()
        if "da" in case:
            assert np.array_equal(a.grad, case["da"]) and np.array_equal(b.grad, case["db"])
    x = mg.Tensor(np.eye(3))
    assert np.array_equal((np.arange(9.0).reshape(3, 3) @ x).data, np.arange(9.0).reshape(3, 3))  # __rmatmul__

    with pytest.raises(ValueError):
        mg.matmul(mg.Tensor(np.ones((2, 3))), 3.0)  # scalars are not allowed
    with pytest.raises(ValueError):
        mg.matmul(mg.Tensor(np.ones((2, 3))), np.ones((4, 2)))  # core dimensions differ
    with pytest.raises(ValueError):
        mg.matmul(mg.Tensor(np.ones((2, 1, 3, 4))), np.ones((3, 2, 4, 5)))  # stacks that do not broadcast
    with pytest.raises(TypeError):
        mg.matmul(mg.Tensor(np.ones((2, 3), dtype=np.int64)), np.ones((3, 2), dtype=np.int64))
    assert mg.matmul(np.ones((0, 3)), np.ones((3, 2))).shape == (0, 2)
    assert np.array_equal(mg.matmul(np.ones((2, 0)), np.ones((0, 3))).data, np.zeros((2, 3)))


def test_dense_layer_chain_stays_on_the_device():
    """relu(x @ w1) @ w2 summed against g: the hidden activations never leave the device."""
    import mygrad_amd as mg
    from mygrad_amd import _device
    from mygrad_amd.nnet import relu

    rng = np.random.default_rng(21)
    x = mg.Tensor(rng.standard_normal((64, 100)))
    w1, w2 = mg.Tensor(rng.standard_normal((100, 80)) * 0.1), mg.Tensor(rng.standard_normal((80, 10)) * 0.1)
    g = rng.standard_normal((64, 10))
    before = dict(_device.stats)
    h = relu(x @ w1)
    out = h @ w2
    h_data = h.data
    out.backward(g)
    assert _device.stats["uploads"] - before["uploads"] == 4  # x, w1, w2 and the seed gradient
    want_h = ora.relu_forward(ora.matmul_forward(x.data, w1.data))
    assert err(h_data, want_h) <= 1e-10
    dh = ora.relu_backward(x.data @ w1.data, ora.matmul_backward(g, want_h, w2.data, 0))
    assert err(w2.grad, ora.matmul_backward(g, want_h, w2.data, 1)) <= 1e-10
    assert err(w1.grad, ora.matmul_backward(dh, x.data, w1.data, 1)) <= 1e-10
    assert err(x.grad, ora.matmul_backward(dh, x.data, w1.data, 0)) <= 1e-10


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shapes", [
    [(10, 100), (100, 5), (5, 50)], [(3, 4), (4, 5), (5, 6), (6, 2)], [(4,), (4, 5), (5, 3)], [(3, 4), (4, 5), (5,)],
    [(4,), (4, 6), (6, 5), (5,)], [(7, 2), (2, 9), (9, 1), (1, 8), (8, 3)], [(3, 4), (4, 5)],
])
def test_multi_matmul_and_its_gradients(shapes, dtype):
    """Same bar as the single product; the expected values are NumPy's chained product and the
    chain rule through the restated matmul gradients, in float64."""
    import mygrad_amd as mg

    dtype = np.dtype(dtype)
    rng = np.random.default_rng([len(shapes), sum(int(np.prod(s)) for s in shapes)])
    arrays = [rng.standard_normal(s).astype(dtype) for s in shapes]
    tensors = [mg.Tensor(a) for a in arrays]
    out = mg.multi_matmul(tensors)
    wide = [a.astype(np.float64) for a in arrays]
    want = wide[0]
    for w in wide[1:]:
        want = ora.matmul_forward(want, w)
    assert out.shape == want.shape and out.dtype == dtype and err(out.data, want) <= TOL[dtype]
    g = rng.standard_normal(want.shape).astype(dtype)
    out.backward(g)
    # d out / d A_i = (A_0 ... A_{i-1})^T g (A_{i+1} ... A_n)^T, by the chain rule from the left
    for i, t in enumerate(tensors):
        left = None
        for w in wide[:i]:
            left = w if left is None else ora.matmul_forward(left, w)
        right = None
        for w in wide[i + 1:]:
            right = w if right is None else ora.matmul_forward(right, w)
        grad = g.astype(np.float64)
        chain = wide[i] if right is None else ora.matmul_forward(wide[i], right)
        if left is not None:
            grad = ora.matmul_backward(grad, left, chain, 1)  # through left @ (A_i right)
        if right is not None:
            grad = ora.matmul_backward(grad, wide[i], right, 0)  # through A_i @ right
        assert t.grad.shape == t.shape and err(t.grad, grad) <= TOL[dtype]
