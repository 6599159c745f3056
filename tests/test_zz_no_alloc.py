"""GPU: the allocation-free scan (ssr_inclusive_sum_i64_static, block sums in a device array inside
the library) gives the bits of ssr_inclusive_sum_i64 with caller scratch, on two calls in a row of
which the second is smaller, and refuses what its workspace cannot hold."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def L(pkg):
    from spirula_studio_amd import lib
    l = lib.load()
    if l.ssr_device_count() < 1:
        pytest.skip("no GPU")
    lib.check(l.ssr_init(0))
    return lib


def _with_scratch(L, a):
    lib = L.load()
    n = a.size
    da, do, tot = L.DeviceArray.from_host(a), L.DeviceArray((n,), np.int64), L.DeviceArray((1,), np.int64)
    sb = lib.ssr_scan_scratch_bytes(n)
    scratch = L.DeviceArray((max(sb, 8),), np.uint8)
    L.check(lib.ssr_inclusive_sum_i64(da.ptr, do.ptr, n, tot.ptr, scratch.ptr, sb, None))
    return do.to_host(), tot.to_host()[0]


def _static(L, a):
    lib = L.load()
    n = a.size
    da, do, tot = L.DeviceArray.from_host(a), L.DeviceArray((n,), np.int64), L.DeviceArray((1,), np.int64)
    L.check(lib.ssr_inclusive_sum_i64_static(da.ptr, do.ptr, n, tot.ptr, None))
    return do.to_host(), tot.to_host()[0]


def test_static_scan_matches_the_scratch_scan_twice(L):
    rng = np.random.default_rng(77)
    # 3 000 017 elements use 1465 block sums; the second call uses 5 of them and must not see the rest. 8 388 609
    # elements are 4097 blocks, one more than a workgroup adds up for itself: the spine kernel then rewrites the
    # static array in place, and the smaller call after it must see nothing of that either.
    for n in (3_000_017, 9_001, 8_388_609, 70_001):
        a = rng.integers(0, 1 << 20, n, dtype=np.int64)
        a[::5] = 0
        a[3] = 1 << 41   # beyond 32 bits
        want, want_total = _with_scratch(L, a)
        got, got_total = _static(L, a)
        assert np.array_equal(want, np.cumsum(a))
        assert np.array_equal(got, want), n
        assert got_total == want_total == int(a.sum())


def test_static_scan_limits(L):
    lib = L.load()
    assert lib.ssr_inclusive_sum_i64_static(None, None, 0, None, None) == 0            # empty: nothing to do
    assert lib.ssr_inclusive_sum_i64_static(8, 8, (1 << 27) + 1, None, None) != 0     # beyond the workspace: refused before any launch
    assert b"2^27" in lib.ssr_last_error()
    assert lib.ssr_inclusive_sum_i64_static(None, None, 5, None, None) != 0 and b"null pointer" in lib.ssr_last_error()
