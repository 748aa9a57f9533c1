"""The allocation-free entry point ah_sum_sq_static against ah_sum_sq, through the C ABI: same inputs, bit-identical
outputs (f32 results of the same partition of f64 partial sums), on two calls in a row, the second with a smaller input,
and no device allocation during the calls."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_sum_sq_static_equals_sum_sq_and_allocates_nothing():
    from alpha2_amd import _ffi as ffi
    lib = ffi.load()
    ffi.check(lib.ah_init(0))

    def alloc(nbytes):
        p = C.c_uint64()
        ffi.check(lib.ah_alloc(nbytes, C.byref(p)))
        return p.value

    def stats():
        s = ffi.AhStats()
        ffi.check(lib.ah_stats(C.byref(s)))
        return s
    rs = np.random.RandomState(3)
    big, small = 5_000_003, 70_001                      # the second call reads fewer partial sums than the first wrote
    x = (rs.randn(big) * 3).astype(np.float32)
    px, out = alloc(big * 4), alloc(16)
    ffi.check(lib.ah_upload(px, x.ctypes.data_as(C.c_void_p), x.nbytes))
    got = np.zeros(4, np.float32)
    want = []
    for n in (big, small):                              # the pool-scratch entry point first (it may allocate)
        ffi.check(lib.ah_sum_sq(px, n, out))
        ffi.check(lib.ah_download(got.ctypes.data_as(C.c_void_p), out, 4))
        want.append(got[0].copy())
        assert abs(float(got[0]) - float(np.sum(x[:n].astype(np.float64) ** 2))) <= 1e-6 * float(got[0])
    before = stats()
    for n, w in zip((big, small), want):
        ffi.check(lib.ah_fill_f32(out, -1.0, 4))
        ffi.check(lib.ah_sum_sq_static(px, n, out + 4))
        ffi.check(lib.ah_download(got.ctypes.data_as(C.c_void_p), out, 16))
        assert got[1].tobytes() == w.tobytes(), (n, got[1], w)          # bit for bit
        assert got[0] == -1.0 and got[2] == -1.0                        # neighbours untouched
    after = stats()
    assert (after.device_mallocs, after.live_allocs, after.pool_blocks) == (before.device_mallocs, before.live_allocs, before.pool_blocks)
    # one element; and sizes it refuses
    ffi.check(lib.ah_sum_sq_static(px, 1, out))
    ffi.check(lib.ah_download(got.ctypes.data_as(C.c_void_p), out, 4))
    assert got[0] == np.float32(np.float64(x[0]) ** 2)
    assert lib.ah_sum_sq_static(px, (1 << 32) + 1, out) == 2 and b"exceeds the maximum" in lib.ah_last_error()
    assert lib.ah_sum_sq_static(px, 0, out) == 2
    lib.ah_free(px), lib.ah_free(out)
