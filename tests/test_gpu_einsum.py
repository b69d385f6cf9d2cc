"""Einstein summation on the device against the NumPy restatement of the reference
(``np.einsum`` forward; the reference's gradient rule), through ``Tensor.backward()``.

Bar (maximum absolute error relative to the largest magnitude of the expected array):
1e-10 in float64, 2e-4 in float32 -- the bar of the matrix product it runs on.  Pure
rearrangements (a transpose, an outer product with a scalar) are exact."""

import numpy as np
import pytest

from oracle import np_oracle as ora

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 2e-4, np.dtype(np.float64): 1e-10}


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    import mygrad_amd as mg

    if not mg.is_available():
        pytest.fail("libmygrad_hip.so / gfx950 device not available: the GPU tests need both")


def err(got, want):
    want = np.asarray(want, dtype=np.float64)
    scale = float(np.max(np.abs(want))) if want.size else 1.0
    return float(np.max(np.abs(np.asarray(got, dtype=np.float64) - want), initial=0.0)) / (scale or 1.0)


CASES = [
    ("ij,jk->ik", [(3, 4), (4, 5)]), ("ij,kj->ik", [(3, 4), (5, 4)]), ("ji,jk->ik", [(4, 3), (4, 5)]),
    ("bij,bjk->bik", [(2, 3, 4), (2, 4, 5)]), ("bji,bjk->bik", [(3, 4, 5), (3, 4, 6)]), ("bij,bkj->bik", [(3, 5, 4), (3, 6, 4)]),
    ("bji,bkj->bki", [(6, 20, 17), (6, 9, 20)]), ("bij,bjk->bik", [(2, 800, 810), (2, 810, 790)]), ("ijk,jil->kl", [(3, 4, 5), (4, 3, 2)]), ("i,i->", [(6,), (6,)]),
    ("i,j->ji", [(3,), (4,)]), ("ij->ji", [(3, 4)]), ("ijk->j", [(2, 3, 4)]), ("ij,jk->i", [(3, 4), (4, 5)]),
    ("ij,k->", [(2, 3), (4,)]), ("abc,cd->dab", [(2, 3, 4), (4, 5)]), (",ij->ij", [(), (2, 3)]),
    ("aib,ajb->abij", [(2, 3, 4), (2, 5, 4)]), ("ij->", [(3, 4)]), ("ij->ij", [(2, 3)]), ("ijkl->lkji", [(2, 3, 4, 5)]),
    ("bhqd,bhkd->bhqk", [(2, 3, 16, 8), (2, 3, 12, 8)]), ("nchw,fc->nfhw", [(2, 16, 5, 5), (8, 16)]),
    ("ij,jk->ik", [(128, 256), (256, 64)]), ("ab,ab->", [(7, 9), (7, 9)]), ("ab,ab->ab", [(7, 9), (7, 9)]),
    ("i,i->i", [(5,), (5,)]), ("ij,j->i", [(0, 3), (3,)]), ("ij,jk->ik", [(2, 0), (0, 3)]),
    # the arrangements that leave the large operand in place: a one-element-window convolution,
    # its input gradient and its filter gradient
    ("nchw,fc->nfhw", [(3, 16, 6, 5), (8, 16)]), ("nfhw,fc->nchw", [(3, 8, 6, 5), (8, 16)]), ("nfhw,nchw->fc", [(3, 8, 6, 5), (3, 16, 6, 5)]),
    ("nfhw,nchw->cf", [(3, 8, 6, 5), (3, 16, 6, 5)]), ("fc,nchw->nfhw", [(8, 16), (3, 16, 6, 5)]),
    # and ones that fit neither: a long scattered sum (filter-gradient kernels), a tall result (roles swapped)
    ("iaj,jbi->ab", [(40, 2, 30), (30, 3, 40)]), ("ai,ib->ba", [(50, 4), (4, 3)]), ("ij,j->i", [(300, 7), (7,)]),
    ("j,jk->k", [(9,), (9, 4)]),
    # more than two operands: contracted pairwise from the left
    ("ij,jk,kl->il", [(3, 4), (4, 5), (5, 2)]), ("bi,bj,bk->ijk", [(4, 2), (4, 3), (4, 5)]), ("i,ij,j->", [(3,), (3, 4), (4,)]),
    ("ab,bc,cd,da->", [(2, 3), (3, 4), (4, 5), (5, 2)]),
    # a label twice within an operand: traces and diagonals
    ("ii->", [(4, 4)]), ("ii->i", [(4, 4)]), ("iji->j", [(3, 2, 3)]), ("ijikik->jk", [(2, 3, 2, 4, 2, 4)]), ("ii,ij->j", [(3, 3), (3, 4)]),
    ("ijj,jk->ik", [(2, 3, 3), (3, 4)]), ("iij->", [(3, 3, 2)]), ("bii->b", [(70, 65, 65)]), ("ii,jj->ij", [(3, 3), (4, 4)]),
    # an axis of length one broadcast against a longer one under the same label
    ("ij,ij->ij", [(2, 3), (1, 3)]), ("bij,bjk->bik", [(1, 3, 4), (5, 4, 2)]), ("bij,bjk->bik", [(5, 3, 4), (1, 4, 2)]),
    ("ai,ai->a", [(4, 1), (4, 6)]), ("ij,jk->ik", [(3, 1), (4, 5)]),
    # both at once: a diagonal of length one under a label that is longer elsewhere
    ("ii,ij->j", [(1, 1), (3, 4)]), ("iji,ik->jk", [(1, 3, 1), (4, 2)]), ("ii,jj->ij", [(1, 1), (4, 4)]), ("iij,ik->jk", [(1, 1, 5), (6, 2)]),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("subscripts, shapes", CASES)
def test_einsum_and_its_gradients_match_the_oracle(subscripts, shapes, dtype):
    import mygrad_amd as mg

    dtype = np.dtype(dtype)
    rng = np.random.default_rng([len(subscripts), sum(int(np.prod(s)) for s in shapes)])
    arrays = [rng.standard_normal(s).astype(dtype) for s in shapes]
    tensors = [mg.Tensor(a) for a in arrays]
    out = mg.einsum(subscripts, *tensors)
    in_lbls, out_lbls = subscripts.split("->")
    wide = [a.astype(np.float64) for a in arrays]
    want = ora.einsum_forward(in_lbls, out_lbls, *wide)
    assert out.shape == want.shape and out.dtype == dtype
    assert err(out.data, want) <= TOL[dtype]
    g = rng.standard_normal(want.shape).astype(dtype)
    out.backward(g)
    for index, t in enumerate(tensors):
        back = ora.einsum_backward(g.astype(np.float64), index, in_lbls, out_lbls, wide)
        assert t.grad.shape == t.shape and t.grad.dtype == dtype
        assert err(t.grad, back) <= TOL[dtype]


def test_reference_docstring_vectors_in_both_calling_conventions(kats):
    import mygrad_amd as mg

    def operand(text):
        return np.asarray(eval(text, {"arange": lambda n: np.arange(float(n))}), dtype=np.float64)  # noqa: S307

    for case in kats["einsum"]:
        got = mg.einsum(case["subscripts"], *[operand(t) for t in case["operands"]])
        assert np.array_equal(got.data, np.array(case["out"], dtype=float)), case["source"]
    a, b = np.arange(60.0).reshape(3, 4, 5), np.arange(24.0).reshape(4, 3, 2)
    got = mg.einsum(mg.Tensor(a), [0, 1, 2], mg.Tensor(b), [1, 0, 3], [2, 3])
    assert np.array_equal(got.data, [[4400, 4730], [4532, 4874], [4664, 5018], [4796, 5162], [4928, 5306]])
    sq = mg.Tensor(np.arange(25.0).reshape(5, 5))
    assert float(mg.einsum("ii", sq).data) == 60.0  # the docstring's trace
    diag = mg.einsum("ii->i", sq)
    assert np.array_equal(diag.data, [0, 6, 12, 18, 24])
    diag.backward(np.arange(5.0))
    assert np.array_equal(sq.grad, np.diag(np.arange(5.0)))
    # rearrangements are copies of values: exact, and never a view of the operand
    c = mg.Tensor(np.arange(6.0).reshape(2, 3))
    t = mg.einsum("ij->ji", c)
    assert np.array_equal(t.data, c.data.T) and not np.shares_memory(t.data, c.data)
    t.clear_graph()


def test_a_tensor_that_occurs_twice_gets_one_gradient_scaled_by_two():
    import mygrad_amd as mg

    x = mg.Tensor(np.arange(1.0, 5.0))
    mg.einsum("i,i->", x, x).backward()
    assert np.array_equal(x.grad, 2 * x.data)  # d (x.x) / dx
    y = mg.Tensor(np.arange(6.0).reshape(2, 3))
    mg.einsum("ij,ij->j", y, y).backward(np.array([1.0, 10.0, 100.0]))
    assert np.array_equal(y.grad, 2 * y.data * np.array([1.0, 10.0, 100.0]))
    w = mg.Tensor(np.arange(1.0, 4.0))
    mg.einsum("i,i,i->", w, w, w).backward()
    assert np.array_equal(w.grad, 3 * w.data**2)
    # the same tensor under different labels is two different pairs
    z = mg.Tensor(np.arange(4.0).reshape(2, 2))
    mg.einsum("ij,jk->ik", z, z).backward()
    want = ora.einsum_backward(np.ones((2, 2)), 0, "ij,jk", "ik", [z.data, z.data]) + ora.einsum_backward(
        np.ones((2, 2)), 1, "ij,jk", "ik", [z.data, z.data])
    assert np.array_equal(z.grad, want)


def test_errors_and_what_is_refused():
    import mygrad_amd as mg

    a, b = mg.Tensor(np.ones((2, 3))), mg.Tensor(np.ones((3, 4)))
    with pytest.raises(ValueError):
        mg.einsum("ij,jk->ik", a, mg.Tensor(np.ones((4, 4))))  # lengths of j differ
    with pytest.raises(ValueError):
        mg.einsum("ijk,jk->i", a, b)  # three labels for two axes
    with pytest.raises(ValueError):
        mg.einsum("ij,jk->ii", a, b)
    with pytest.raises(ValueError):
        mg.einsum("ii->i", mg.Tensor(np.ones((3, 4))))  # the two axes of a diagonal differ in length
    with pytest.raises(ValueError):
        mg.einsum("ii,ij->j", mg.Tensor(np.ones((3, 1))), mg.Tensor(np.ones((3, 2))))  # one axis of the diagonal broadcast, one not
    with pytest.raises(TypeError):
        mg.einsum("ij,jk->ik", mg.Tensor(np.ones((2, 3), dtype=np.int64)), mg.Tensor(np.ones((3, 4), dtype=np.int64)))


def test_one_element_window_convolution_full_size():
    """The benchmark's summation, 'nchw,fc->nfhw' on (32,256,56,56) x (256,256) with both
    gradients, against BLAS products of the same operands in float64 (2e-4 bar)."""
    import mygrad_amd as mg

    rng = np.random.default_rng(95)
    xv = rng.standard_normal((32, 256, 56, 56), dtype=np.float32)
    wv = (rng.standard_normal((256, 256)) / 16).astype(np.float32)
    x, w = mg.Tensor(xv), mg.Tensor(wv)
    out = mg.einsum("nchw,fc->nfhw", x, w)
    x64, w64 = xv.astype(np.float64), wv.astype(np.float64)
    want = np.tensordot(w64, x64, axes=([1], [1])).transpose(1, 0, 2, 3)
    assert err(out.data, want) <= 2e-4
    g = rng.standard_normal(out.shape, dtype=np.float32)
    out.backward(g)
    g64 = g.astype(np.float64)
    assert err(x.grad, np.tensordot(w64, g64, axes=([0], [1])).transpose(1, 0, 2, 3)) <= 2e-4
    assert err(w.grad, np.tensordot(g64, x64, axes=([0, 2, 3], [0, 2, 3]))) <= 2e-4


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_out_receives_the_result_and_becomes_the_data(dtype):
    """``einsum(..., out=array)`` (reference: mygrad/linalg/funcs.py:445-451 hands the array to
    ``np.einsum`` through ``Tensor._op``, mygrad/tensor_base.py:1110-1113): the array is written,
    it is the returned tensor's data, and back-propagation runs as without it."""
    import mygrad_amd as mg

    rng = np.random.default_rng(31)
    a, b = rng.standard_normal((6, 7)).astype(dtype), rng.standard_normal((7, 5)).astype(dtype)
    want = a.astype(np.float64) @ b.astype(np.float64)
    ta, tb = mg.Tensor(a), mg.Tensor(b)
    target = np.full((6, 5), np.nan, dtype=dtype)
    res = mg.einsum("ij,jk->ik", ta, tb, out=target)
    assert res.data is target and err(target, want) <= TOL[np.dtype(dtype)]
    plain = mg.einsum("ij,jk->ik", a, b)
    assert np.array_equal(target, plain.data)
    g = rng.standard_normal((6, 5)).astype(dtype)
    res.backward(g)
    assert err(ta.grad, g.astype(np.float64) @ b.T.astype(np.float64)) <= TOL[np.dtype(dtype)]
    assert err(tb.grad, a.T.astype(np.float64) @ g.astype(np.float64)) <= TOL[np.dtype(dtype)]
    # a consumer of the result reads the same values (from the device copy or from the array)
    twice = mg.einsum("ik->ki", res)
    assert np.array_equal(twice.data, target.T)

    # a strided target and a wider one are filled through the host
    wide = np.zeros((5, 6), dtype=np.float64).T
    assert mg.einsum("ij,jk->ik", a, b, out=wide).data is wide
    assert np.array_equal(wide, plain.data.astype(np.float64))
    # an empty sum writes zeros
    empty = np.full((2, 3), 7.0, dtype=dtype)
    mg.einsum("ij,jk->ik", np.ones((2, 0), dtype=dtype), np.ones((0, 3), dtype=dtype), out=empty)
    assert np.array_equal(empty, np.zeros((2, 3)))
