"""SeededRng (packages/core/src/rng.ts:6-68) over the library's host-side implementation."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _ffi as ffi


def _i32(x: int) -> int:
    x &= 0xFFFFFFFF
    return x - (1 << 32) if x >= (1 << 31) else x


class SeededRng:
    def __init__(self, seed: int = 42):
        self._lib = ffi.load()
        self._s = ffi.AhRng()
        self.seed(seed)

    def seed(self, s: int):
        self._seed = s
        ffi.check(self._lib.ah_rng_seed(C.byref(self._s), _i32(s)))

    def state(self) -> int:
        return self._seed

    def setState(self, s: int):
        self.seed(s)

    def next(self) -> float:
        out = C.c_double()
        ffi.check(self._lib.ah_rng_next(C.byref(self._s), C.byref(out)))
        return out.value

    def nextGauss(self) -> float:
        out = C.c_double()
        ffi.check(self._lib.ah_rng_next_gauss(C.byref(self._s), C.byref(out)))
        return out.value

    def fillGauss(self, n: int, std: float) -> np.ndarray:
        """n draws of nextGauss()*std rounded to f32 (initWeight, packages/model/src/gpt.ts:53-59)."""
        out = np.empty(n, dtype=np.float32)
        ffi.check(self._lib.ah_rng_fill_gauss_f32(C.byref(self._s), out.ctypes.data_as(C.c_void_p), n, std))
        return out

    def fillUniform(self, n: int) -> np.ndarray:
        out = np.empty(n, dtype=np.float64)
        ffi.check(self._lib.ah_rng_fill_uniform_f64(C.byref(self._s), out.ctypes.data_as(C.c_void_p), n))
        return out
