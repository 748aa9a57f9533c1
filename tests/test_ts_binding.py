"""The TypeScript package a maintainer of the reference would add (integration/hip/src/*.ts) cannot be compiled in this
image (no bun / tsc), so it is tied to the library mechanically: the `dlopen` table of ffi.ts is parsed and compared,
symbol by symbol, with the header and with the ctypes table the GPU tests call through (names, argument counts, argument
and return types); the struct layouts it fills by hand are compared with ctypes' offsets; every `lib.ah_*(...)` call in
backend.ts must pass as many arguments as its table entry takes; and the class must define every member of the reference's
`Backend` interface and the duck-typed extras its trainer calls."""
import ctypes as C
import json
import os
import re

from alpha2_amd import _ffi as ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "integration", "hip", "src")
SCALAR = {C.c_int32: "i32", C.c_uint64: "u64", C.c_int64: "i64", C.c_float: "f32", C.c_double: "f64"}


def _read(name):
    return open(os.path.join(SRC, name)).read()


def _table():
    body = _read("ffi.ts").split("dlopen(", 1)[1].split("}).symbols", 1)[0]
    rows = re.findall(r"^\s*(ah_[a-z0-9_]+):\s*\{\s*args:\s*\[([^\]]*)\],\s*returns:\s*(\w+)\s*\}", body, flags=re.M)
    return {n: ([a.strip() for a in args.split(",") if a.strip()], ret) for n, args, ret in rows}


def _header_symbols():
    src = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "alpha_hip.h")).read(), flags=re.S)
    decl = {}
    for ret, name, args in re.findall(r"^\s*([A-Za-z_][\w \*]*?)\s*\b(ah_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", src, flags=re.M):
        args = args.strip()
        decl[name] = (ret.strip(), [] if args in ("", "void") else [a.strip() for a in args.split(",")])
    return decl


def test_dlopen_table_binds_exactly_the_header_with_the_argument_types_of_the_ctypes_table():
    table, decl = _table(), _header_symbols()
    assert len(table) > 100 and set(table) == set(decl), (set(table) - set(decl), set(decl) - set(table))
    for name, (args, ret) in table.items():
        c_ret, c_args = decl[name]
        assert len(args) == len(c_args), (name, args, c_args)
        for ts, c in zip(args, c_args):             # against the header: pointers are pointers, scalars have the C type's width
            if "*" in c:
                assert ts == "ptr", (name, ts, c)
            else:
                ctype = c.split()[0] if not c.startswith("const ") else c.split()[1]
                want = {"int32_t": "i32", "int64_t": "i64", "uint64_t": "u64", "ah_ptr": "u64", "float": "f32", "double": "f64"}[ctype]
                assert ts == want, (name, ts, c)
        if name in ffi.SIGNATURES:                  # against the table the GPU tests call through
            assert args == [SCALAR.get(t, "ptr") for t in ffi.SIGNATURES[name]], name
        want_ret = "cstring" if "char" in c_ret else {"int32_t": "i32", "int64_t": "i64"}[c_ret]
        assert ret == want_ret, (name, ret, c_ret)


def test_struct_layouts_written_by_hand_in_typescript_are_the_c_layouts():
    body = _read("ffi.ts").split("export const LAYOUT = {", 1)[1].split("} as const", 1)[0]
    rows = re.findall(r"^\s*(Ah\w+):\s*\{([^}]*)\}", body, flags=re.M)
    assert {n for n, _ in rows} >= {"AhGemm", "AhFlash", "AhAdamW", "AhStats", "AhDeviceInfo"}
    for name, fields in rows:
        cls = getattr(ffi, name)
        got = {k.strip(): int(v) for k, v in (f.split(":") for f in fields.split(",") if f.strip())}
        assert got.pop("size") == C.sizeof(cls), name
        assert got == {n: getattr(cls, n).offset for n, _ in cls._fields_}, name
    # ... and the fields backend.ts sets on them exist, with a setter of the field's C type
    setter = {C.c_int32: "i32", C.c_float: "f32", C.c_double: "f64", C.c_int64: "i64", C.c_uint64: "u64"}
    src = _read("backend.ts")
    for var, cls in (("g", ffi.AhGemm), ("f", ffi.AhFlash), ("a", ffi.AhAdamW)):
        types = dict(cls._fields_)
        for kind, field in re.findall(r"\b%s\.(i32|f32|f64|i64|u64)\(\"(\w+)\"" % var, src):
            assert field in types and setter[types[field]] == kind, (cls.__name__, field, kind)
    for kind, suffix in re.findall(r"f\.(i64)\(p \+ \"(_\w+)\"", src):
        assert all(dict(ffi.AhFlash._fields_)[p + suffix] is C.c_int64 for p in "qkvo")


def _call_arg_counts(src):
    for m in re.finditer(r"\blib\.(ah_[a-z0-9_]+)\(", src):
        depth, i, n, seen = 1, m.end(), 0, False
        while depth:
            ch = src[i]
            if ch in "([{":
                depth += 1
            elif ch in ")]}":
                depth -= 1
            elif ch == "," and depth == 1:
                n += 1
            if depth and not ch.isspace():
                seen = True
            i += 1
        yield m.group(1), (n + 1 if seen else 0)


def test_every_library_call_of_the_backend_class_passes_the_arguments_its_entry_takes():
    table = _table()
    calls = list(_call_arg_counts(_read("backend.ts"))) + list(_call_arg_counts(_read("ffi.ts")))
    assert len(calls) > 50
    for name, n in calls:
        assert name in table and n == len(table[name][0]), (name, n, table.get(name))


def test_backend_class_defines_every_member_of_the_reference_interface_and_registers_as_hip():
    spec = json.load(open(os.path.join(ROOT, "tests", "golden", "backend_interface.json")))
    src = _read("backend.ts")
    assert re.search(r"export class HipBackend implements Backend\b", src) and re.search(r'readonly name = "hip"', src)
    members = set(re.findall(r"^  (?:get )?([a-zA-Z]\w*)\s*\(", src, flags=re.M))
    missing = [n for n in spec["required"][1:] + spec["optional"] + spec["duck_typed"] if n not in members]
    assert not missing, missing
    assert "smokeTest" not in members                   # trainer.ts:623: the smoke-test path is for NVIDIA devices
    idx = _read("index.ts")
    assert re.search(r'new Registry<Backend>\("backend"\)', idx) and re.search(r'register\("hip",\s*\(\)\s*=>\s*new HipBackend\(\)\)', idx)
