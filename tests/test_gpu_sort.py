"""GPU: the radix sort and the int64 scan through the C ABI against exact CPU answers -- the method
of src/backend/vulkan/tests/vk_sortscan_test.cpp (std::stable_sort on the masked key :67-80, the
size ladder and tile-key bit ranges :185-201, duplicate-heavy keys :199, serial scan :113-148)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def L(pkg):
    from spirula_studio_amd import lib
    lib.check(lib.load().ssr_init(0))
    return lib


def _sort(L, keys, vals, b0, b1):
    lib = L.load()
    n = keys.size
    ka, kb = L.DeviceArray.from_host(keys), L.DeviceArray((n,), np.int64)
    va, vb = L.DeviceArray.from_host(vals), L.DeviceArray((n,), np.int32)
    sb = lib.ssr_sort_scratch_bytes(n)
    scratch = L.DeviceArray((max(sb, 16),), np.uint8)
    sel = C.c_int(-1)
    L.check(lib.ssr_sort_pairs_u64_i32(ka.ptr, kb.ptr, va.ptr, vb.ptr, n, b0, b1, C.byref(sel), scratch.ptr, sb, None))
    k, v = (kb, vb) if sel.value else (ka, va)
    return k.to_host(), v.to_host()


@pytest.mark.parametrize("n", [0, 1, 2, 63, 64, 65, 4095, 4096, 4097, 100003, (1 << 20) + 123, 5_000_001])
@pytest.mark.parametrize("bits", [(0, 44), (0, 49), (0, 64), (8, 24), (3, 4)])
def test_sort_pairs(L, n, bits):
    if n > 200000 and bits not in [(0, 44), (0, 49)]:
        pytest.skip("large sizes on the tile-key bit ranges only")
    rng = np.random.default_rng(n * 7 + bits[1])
    keys = rng.integers(0, 1 << 62, n, dtype=np.int64)
    if n > 100:
        keys[: n // 2] &= 0xFF                      # duplicate-heavy half
        keys[n // 2: n // 2 + n // 8] = keys[0]     # one long run of a single key
    vals = rng.integers(-(1 << 31), 1 << 31, n, dtype=np.int64).astype(np.int32)
    ko, vo = _sort(L, keys, vals, *bits)
    nb = bits[1] - bits[0]
    mask = np.uint64(0xFFFFFFFFFFFFFFFF) if nb >= 64 else np.uint64(((1 << nb) - 1) << bits[0])
    order = np.argsort(keys.view(np.uint64) & mask, kind="stable")
    assert np.array_equal(ko, keys[order])
    assert np.array_equal(vo, vals[order])


def test_sort_already_sorted_and_reversed(L):
    n = 300001
    keys = (np.arange(n, dtype=np.int64) << 13)
    vals = np.arange(n, dtype=np.int32)
    ko, vo = _sort(L, keys, vals, 0, 45)
    assert np.array_equal(ko, keys) and np.array_equal(vo, vals)
    ko, vo = _sort(L, keys[::-1].copy(), vals, 0, 45)
    assert np.array_equal(ko, keys) and np.array_equal(vo, vals[::-1])


@pytest.mark.parametrize("n", [1, 2, 255, 256, 2047, 2048, 2049, 1_000_003, 10_000_019])
def test_inclusive_sum_i64(L, n):
    lib = L.load()
    rng = np.random.default_rng(n)
    a = rng.integers(0, 1 << 20, n, dtype=np.int64)
    if n > 1000:
        a[::7] = 0
        a[5] = 1 << 40   # beyond 32 bits
    da, do, tot = L.DeviceArray.from_host(a), L.DeviceArray((n,), np.int64), L.DeviceArray((2,), np.int64)
    sb = lib.ssr_scan_scratch_bytes(n)
    scratch = L.DeviceArray((max(sb, 8),), np.uint8)
    L.check(lib.ssr_inclusive_sum_i64(da.ptr, do.ptr, n, tot.ptr, scratch.ptr, sb, None))
    want = np.cumsum(a)
    assert np.array_equal(do.to_host(), want)
    assert tot.to_host()[0] == want[-1]
    # in place
    L.check(lib.ssr_inclusive_sum_i64(da.ptr, da.ptr, n, None, scratch.ptr, sb, None))
    assert np.array_equal(da.to_host(), want)


def test_argument_errors(L):
    lib = L.load()
    sel = C.c_int(0)
    assert lib.ssr_sort_pairs_u64_i32(None, None, None, None, 10, 0, 8, C.byref(sel), None, 0, None) != 0
    assert b"null buffer" in lib.ssr_last_error()
    assert lib.ssr_sort_pairs_u64_i32(None, None, None, None, 10, 9, 8, C.byref(sel), None, 0, None) != 0
    assert b"bit range" in lib.ssr_last_error()
    assert lib.ssr_inclusive_sum_i64(None, None, 5, None, None, 0, None) != 0
    assert lib.ssr_last_error() != b""
    assert lib.ssr_sort_pairs_u64_i32(None, None, None, None, 0, 0, 8, C.byref(sel), None, 0, None) == 0
