"""CPU-only checks of the C-ABI boundary: the built library loads, exports every symbol the header declares, the
ctypes table binds exactly those symbols, and the host-only entry points behave (no device compute here)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from alpha2_amd import _ffi as ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    src = open(os.path.join(ROOT, "include", "alpha_hip.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(ah_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    lib = C.CDLL(ffi.LIB_PATH)
    names = _declared()
    assert len(names) > 60
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_binding_table_matches_header():
    names = set(_declared())
    bound = set(ffi.SIGNATURES) | {"ah_last_error", "ah_step_note"}
    assert names == bound, (names - bound, bound - names)
    ffi.load()


def test_calls_before_init_fail_with_message_not_crash():
    lib = ffi.load()
    out = C.c_uint64(0)
    rc = lib.ah_alloc(1024, C.byref(out))
    if rc == 0:                       # another test in this process already initialised a device
        lib.ah_free(out.value)
        pytest.skip("device already initialised")
    assert rc == 3 and b"ah_init" in lib.ah_last_error()


def test_host_rng_matches_reference_integer_stream():
    """Independent big-int restatement of packages/core/src/rng.ts:13-50 against the library's host RNG."""
    from alpha2_amd.rng import SeededRng
    M = 0xFFFFFFFF

    def i32(x):
        x &= M
        return x - (1 << 32) if x >> 31 else x
    for seed in (0, 42, -5, 123456789):
        s0, s1 = i32(seed), i32(seed ^ 0xDEADBEEF)
        want = []
        for i in range(120):
            a, b = s0 & M, s1 & M
            s0 = i32(b)
            a ^= (a << 23) & M
            a ^= a >> 17
            a ^= b
            a ^= b >> 26
            s1 = i32(a)
            if i >= 20:
                want.append(((s0 + s1) & M) / 4294967296.0)
        r = SeededRng(seed)
        assert [r.next() for _ in range(100)] == want
    r = SeededRng(7)
    g = r.fillGauss(4001, 0.02)
    assert g.dtype == np.float32 and abs(float(g.mean())) < 2e-3 and abs(float(g.std()) - 0.02) < 2e-3


def test_backend_class_has_every_member_of_the_reference_interface():
    """Member names of the reference's `interface Backend` (the 40 required and 27 optional ones, fixture transcribed
    from packages/core/src/interfaces.ts:38-151) and the duck-typed extras its trainer calls (trainer.ts:1003-1032)."""
    import json
    from alpha2_amd.backend import HipBackend
    spec = json.load(open(os.path.join(ROOT, "tests", "golden", "backend_interface.json")))
    assert len(spec["required"]) == 40 and len(spec["optional"]) == 27
    missing = [n for n in spec["required"] + spec["optional"] + spec["duck_typed"] if not hasattr(HipBackend, n)]
    assert not missing, missing
    assert HipBackend.name == "hip"
