"""ffi/peregrine-hip-sys (the Rust binding a peregrine maintainer would add) against
include/peregrine_hip.h.  The image has no Rust toolchain, so these checks stand in for a
build: the generated `extern "C"` block is current, every declared symbol is bound with the
header's arity, and the Rust types agree with the ctypes table the GPU tests call through."""
import ctypes as C
import importlib.util
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CRATE = os.path.join(ROOT, "ffi", "peregrine-hip-sys")


def _gen():
    spec = importlib.util.spec_from_file_location("gen_bindings", os.path.join(CRATE, "gen_bindings.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _rust_fns():
    """{name: ([argument types], return type or "")} parsed from src/lib.rs's extern block."""
    src = open(os.path.join(CRATE, "src", "lib.rs")).read()
    block = src[src.index('extern "C" {'):]
    block = block[:block.index("\n}")]
    out = {}
    for m in re.finditer(r"pub fn (pg_[a-z0-9_]+)\((.*?)\)(?: -> ([^;]+))?;", block):
        args = [a.split(":", 1)[1].strip() for a in m.group(2).split(", ") if a.strip()]
        out[m.group(1)] = (args, (m.group(3) or "").strip())
    return out


def test_generated_block_is_current():
    g = _gen()
    src = open(g.LIB_RS).read()
    a, b = src.index(g.BEGIN), src.index(g.END) + len(g.END)
    assert src[a:b] == g.generated_block(), "run ffi/peregrine-hip-sys/gen_bindings.py"


def test_every_header_symbol_is_bound_with_its_arity():
    from test_abi_symbols import declared_symbols  # an independent, regex-only reading of the header

    text = open(os.path.join(ROOT, "include", "peregrine_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    rust = _rust_fns()
    names = declared_symbols()
    assert sorted(rust) == names
    for name in names:
        m = re.search(r"\b" + name + r"\s*\(([^;]*?)\)\s*;", text, flags=re.S)
        c_args = m.group(1).strip()
        arity = 0 if c_args in ("", "void") else c_args.count(",") + 1
        assert len(rust[name][0]) == arity, f"{name}: header has {arity} parameters, lib.rs {len(rust[name][0])}"
        returns_void = re.search(r"\bvoid\s+" + name + r"\s*\(", text) is not None
        assert (rust[name][1] == "") == returns_void, name


def test_rust_types_agree_with_the_ctypes_binding():
    from peregrine_amd import _ffi

    scalar = {C.c_size_t: "usize", C.c_int: "c_int", C.c_float: "f32", C.c_double: "f64"}
    rust = _rust_fns()
    assert sorted(rust) == sorted(_ffi.SIGNATURES)
    for name, argtypes in _ffi.SIGNATURES.items():
        rargs, rret = rust[name]
        assert len(rargs) == len(argtypes), name
        for i, (ct, rt) in enumerate(zip(argtypes, rargs)):
            if ct in scalar:
                want = scalar[ct]
                assert rt == want or (want == "c_int" and rt == "pg_status"), f"{name} argument {i}: ctypes {ct.__name__}, rust {rt}"
            else:  # c_void_p, c_char_p, POINTER(...): a pointer on both sides
                assert rt.startswith("*"), f"{name} argument {i}: ctypes pointer, rust {rt}"
        restype = _ffi._OTHER_RESTYPE.get(name, C.c_int)
        want_ret = {None: "", C.c_int: "pg_status", C.c_size_t: "usize", C.c_void_p: "*mut c_void", C.c_char_p: "*const c_char"}[restype]
        assert rret == want_ret, f"{name}: returns {rret!r}, ctypes says {want_ret!r}"


def test_type_mapping_rules():
    g = _gen()
    for c, r in [("const float *", "*const f32"), ("float *", "*mut f32"), ("size_t", "usize"), ("int", "c_int"),
                 ("const pg_gguf_tensor *const *", "*const *const pg_gguf_tensor"), ("float *const *", "*const *mut f32"),
                 ("const char **", "*mut *const c_char"), ("void **", "*mut *mut c_void"), ("pg_qtensor **", "*mut *mut pg_qtensor"),
                 ("const uint8_t *const *", "*const *const u8"), ("const void *", "*const c_void"), ("int32_t *", "*mut i32"),
                 ("const size_t *", "*const usize"), ("void", ""), ("pg_status", "pg_status"), ("const pg_ctx *", "*const pg_ctx")]:
        assert g.rust_type(c) == r, (c, g.rust_type(c), r)


def test_constants_and_opaque_types_match_the_header():
    g = _gen()
    header = open(os.path.join(ROOT, "include", "peregrine_hip.h")).read()
    lib = open(os.path.join(CRATE, "src", "lib.rs")).read()
    for t in g.opaque_types():
        assert re.search(r"opaque!\([^)]*\b" + t + r"\b", lib), f"opaque type {t} missing from lib.rs"
    consts = dict(re.findall(r"\b(PG_[A-Z0-9_]+)\s*=\s*(\d+)", header))
    consts.update(dict(re.findall(r"#define (PG_MASK_[A-Z_]+) (\d+)", header)))
    assert len(consts) >= 14
    for name, value in consts.items():
        m = re.search(r"pub const " + name + r": \w+ = (\d+);", lib)
        assert m and m.group(1) == value, f"{name}: header {value}, lib.rs {m.group(1) if m else None}"
