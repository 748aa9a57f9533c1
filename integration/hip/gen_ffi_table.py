#!/usr/bin/env python3
"""Writes the `dlopen` symbol table and the struct layouts of src/ffi.ts (the part between the GENERATED markers) from
alpha2_amd/_ffi.py, the ctypes table that tests/test_abi.py ties to include/alpha_hip.h.

    python integration/hip/gen_ffi_table.py            # rewrites integration/hip/src/ffi.ts in place
"""
import ctypes as C
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
from alpha2_amd import _ffi as ffi  # noqa: E402

SCALARS = {C.c_int32: "i32", C.c_uint64: "u64", C.c_int64: "i64", C.c_float: "f32", C.c_double: "f64"}
RETURNS = {"ah_last_error": "cstring", "ah_step_note": "cstring", "ah_layernorm_bwd_partials_bytes": "i64", "ah_embedding_index_bytes": "i64"}
STRUCTS = ("AhGemm", "AhFlash", "AhAdamW", "AhAdamWItem", "AhStats", "AhDeviceInfo", "AhColsumJob", "AhLion", "AhAdafactor", "AhRng")


def ts_type(t) -> str:
    return SCALARS.get(t, "ptr")          # every pointer type (typed, void*, char*) crosses as a pointer


def table() -> str:
    names = dict(ffi.SIGNATURES)
    names["ah_last_error"], names["ah_step_note"] = [], []
    width = max(len(n) for n in names) + 1
    lines = []
    for name in sorted(names):
        args = ", ".join(ts_type(t) for t in names[name])
        lines.append(f"  {(name + ':').ljust(width)} {{ args: [{args}], returns: {RETURNS.get(name, 'i32')} }},")
    return "\n".join(lines)


def layouts() -> str:
    out = []
    for s in STRUCTS:
        cls = getattr(ffi, s)
        fields = ", ".join(f"{n}: {getattr(cls, n).offset}" for n, _ in cls._fields_)
        out.append(f"  {s}: {{ size: {C.sizeof(cls)}, {fields} }},")
    return "\n".join(out)


def main():
    path = os.path.join(HERE, "src", "ffi.ts")
    src = open(path).read()
    for tag, body in (("SYMBOLS", table()), ("LAYOUTS", layouts())):
        a, b = f"  // GENERATED {tag} BEGIN\n", f"\n  // GENERATED {tag} END"
        i, j = src.index(a) + len(a), src.index(b)
        src = src[:i] + body + src[j:]
    open(path, "w").write(src)


if __name__ == "__main__":
    main()
