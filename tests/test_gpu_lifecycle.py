"""ah_init / ah_shutdown through the C ABI, in a process of its own (shutting the library down would pull the device
memory from under the other tests' backend): work, shut down, every call then refused with AH_ERR_STATE until the
library is initialised again, work again with nothing left over from the first life (a grouped-GEMM plan made in the first
life is unknown in the second: its tables went with the shutdown)."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SCRIPT = r"""
import ctypes as C
import numpy as np
from alpha2_amd import _ffi as ffi
lib = ffi.load()
assert lib.ah_shutdown() == 0                                   # before any init: nothing to do
p = C.c_uint64()
assert lib.ah_alloc(64, C.byref(p)) == 3 and b"ah_init" in lib.ah_last_error()       # AH_ERR_STATE
x = np.arange(1000, dtype=np.float32)
got = np.zeros(1, np.float32)
old_plan = None
for life in range(2):
    ffi.check(lib.ah_init(0))
    ffi.check(lib.ah_init(0))                                   # a second init of the same device is accepted
    s = ffi.AhStats()
    ffi.check(lib.ah_stats(C.byref(s)))
    assert s.live_allocs == 0, (life, s.live_allocs)
    px, out = C.c_uint64(), C.c_uint64()
    ffi.check(lib.ah_alloc(x.nbytes, C.byref(px)))
    ffi.check(lib.ah_alloc(16, C.byref(out)))
    ffi.check(lib.ah_upload(px.value, x.ctypes.data_as(C.c_void_p), x.nbytes))
    ffi.check(lib.ah_sum_sq(px.value, x.size, out.value))
    ffi.check(lib.ah_sum_sq_static(px.value, x.size, out.value + 4))             # its per-device array is found again after a shutdown
    two = np.zeros(2, np.float32)
    ffi.check(lib.ah_download(two.ctypes.data_as(C.c_void_p), out.value, 8))
    assert two[0] == two[1] == np.float32(float((x.astype(np.float64) ** 2).sum())), two
    if old_plan is not None:                                    # an id from before the shutdown
        assert lib.ah_gemm_grouped_run(old_plan, ffi.EPI_NONE) == 2 and b"unknown plan" in lib.ah_last_error()      # AH_ERR_ARG
        assert lib.ah_gemm_grouped_destroy(old_plan) == 2
    ga, gb, gc = C.c_uint64(), C.c_uint64(), C.c_uint64()       # two 256 x 256 weight gradients over 64 tokens
    ffi.check(lib.ah_alloc(64 * 256 * 2, C.byref(ga))); ffi.check(lib.ah_alloc(64 * 256 * 2, C.byref(gb)))
    ffi.check(lib.ah_alloc(2 * 256 * 256 * 4, C.byref(gc)))
    ffi.check(lib.ah_fill_f32(ga.value, 0.0, 64 * 256 // 2)); ffi.check(lib.ah_fill_f32(gb.value, 0.0, 64 * 256 // 2))
    descs = (ffi.AhGemm * 2)(*[ffi.AhGemm(ffi.GEMM_TN, ffi.BF16, ffi.F32, ffi.EPI_NONE, 256, 256, 64, 256, 256, 256, 1, 0, 0, 0,
                                            ga.value, gb.value, gc.value + i * 256 * 256 * 4, 0) for i in range(2)])
    pid = C.c_uint64()
    ffi.check(lib.ah_gemm_grouped_plan(descs, 2, C.byref(pid)))
    ffi.check(lib.ah_gemm_grouped_run(pid.value, ffi.EPI_NONE))
    assert old_plan is None or pid.value != old_plan
    old_plan = pid.value
    assert lib.ah_shutdown() == 0                               # frees what the caller left allocated
    assert lib.ah_sum_sq(px.value, x.size, out.value) == 3
    assert lib.ah_free(px.value) == 3
print("lifecycle ok")
"""


def test_shutdown_and_a_second_life():
    env = dict(os.environ, PYTHONPATH=ROOT + os.pathsep + os.environ.get("PYTHONPATH", ""))
    r = subprocess.run([sys.executable, "-c", SCRIPT], capture_output=True, text=True, cwd=ROOT, env=env, timeout=100)
    assert r.returncode == 0 and "lifecycle ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
