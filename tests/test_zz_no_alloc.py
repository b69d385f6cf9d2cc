"""mg_sum_all_static, the whole-array sum that allocates nothing, against mg_sum_all: the two
share kernels and chunking, so every result must agree bit for bit -- also on a second call
with a smaller input, which finds the first call's chunk sums still in the shared array."""

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def abi():
    import mygrad_amd

    if not mygrad_amd.is_available():
        pytest.fail("libmygrad_hip.so / gfx950 device not available: the GPU tests need both")
    from tests import abi as module

    return module


def bits(a):
    a = np.asarray(a).reshape(1)
    return a.view(np.uint32 if a.dtype == np.float32 else np.uint64)[0]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_static_sum_matches_the_allocating_entry_point_twice_in_a_row(abi, dtype):
    rng = np.random.default_rng(77)
    # 5 000 003 elements: many chunks and a ragged tail; then 70 001: fewer chunks than before,
    # so stale chunk sums of the first call sit right behind the ones the second call writes
    for n in (5_000_003, 70_001, 3, 1_000_000):
        x = (rng.standard_normal(n) * 10.0 ** rng.integers(-3, 4, n)).astype(dtype)
        want = abi.sum_all(x)
        got = abi.sum_all_static(x)
        assert bits(got) == bits(want), (n, got, want)
        assert bits(abi.sum_all_static(x)) == bits(want)


def test_static_sum_known_values_and_refusals(abi):
    from mygrad_amd import _device, _hip

    n = 1 << 20
    assert float(abi.sum_all_static(np.arange(n, dtype=np.float64))) == n * (n - 1) / 2
    assert float(abi.sum_all_static(np.ones(12345, dtype=np.float32))) == 12345.0
    lib = _hip.lib()
    buf = _device.DeviceBuffer(64)
    assert lib.mg_sum_all_static(1, 0, None, buf.ptr) == 0  # the empty sum
    out = np.empty((), np.float64)
    buf.download_into(out.reshape(1))
    assert float(out) == 0.0
    assert lib.mg_sum_all_static(0, (1 << 31) + 1, buf.ptr, buf.ptr) == -2  # beyond the stated maximum
    assert b"exceeds" in lib.mg_last_error()
    assert lib.mg_sum_all_static(1, 4, buf.ptr + 8, buf.ptr) == -1  # misaligned
    assert lib.mg_sum_all_static(5, 4, buf.ptr, buf.ptr) == -2  # dtype
