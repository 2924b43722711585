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


# The public functions of `peregrine::quant` and `peregrine::gguf` on this path, as the reference declares them
# (name -> normalised "(parameter types) -> return type").  `self` receivers keep their form.
REFERENCE_SIGNATURES = {
    # /root/reference/src/quant.rs:27, 79, 115, 129-134, 174, 183, 196-202
    "quant::quantize_weights": "(&[f32], usize, usize) -> QuantizedTensor",
    "quant::quantize_activations": "(&[f32], usize, usize) -> (Vec<i8>, Vec<f32>)",
    "quant::dequantize": "(&QuantizedTensor) -> Vec<f32>",
    "quant::matmul_quantized": "(&[f32], usize, usize, &QuantizedTensor) -> Vec<f32>",
    "quant::to_gpu": "(&mut self, &GpuContext)",
    "quant::from_gpu": "(&mut self, &GpuContext)",
    "quant::matmul_quantized_gpu": "(&GpuContext, &[f32], usize, usize, &QuantizedTensor) -> GpuBuffer<f32>",
    # /root/reference/src/gguf.rs:286, 307, 331, 354, 386-390
    "gguf::dequant_q8_0": "(&[u8], usize) -> Vec<f32>",
    "gguf::dequant_q4_0": "(&[u8], usize) -> Vec<f32>",
    "gguf::dequant_q4_1": "(&[u8], usize) -> Vec<f32>",
    "gguf::f16_to_f32": "(u16) -> f32",
    "gguf::load_tensor_q8_as_quantized": "(&[u8], usize, usize) -> crate::quant::QuantizedTensor",
}


def _pub_fn_signatures(src):
    """{name: "(types) -> ret"} of every `pub fn` in a piece of Rust source (parameter names dropped)."""
    out = {}
    for m in re.finditer(r"pub fn (\w+)\s*\((.*?)\)\s*(?:->\s*(.*?))?\s*\{", src, flags=re.S):
        params = []
        depth, cur = 0, ""
        for ch in m.group(2):  # split on top-level commas only
            if ch in "<([":
                depth += 1
            elif ch in ">)]":
                depth -= 1
            if ch == "," and depth == 0:
                params.append(cur)
                cur = ""
            else:
                cur += ch
        params.append(cur)
        types = []
        for p in (q.strip() for q in params):
            if not p:
                continue
            types.append(p if "self" in p.split(":")[0] and ":" not in p else " ".join(p.split(":", 1)[1].split()))
        sig = "(" + ", ".join(types) + ")"
        if m.group(3):
            sig += " -> " + " ".join(m.group(3).split())
        out.setdefault(m.group(1), sig)
    return out


def _module(src, name):
    a = src.index(f"pub mod {name} {{")
    b = src.index("\n}\n", a)
    return src[a:b]


def test_quant_and_gguf_wrappers_keep_the_reference_signatures():
    src = open(os.path.join(CRATE, "src", "lib.rs")).read()
    ours = {}
    for mod in ("quant", "gguf"):
        for name, sig in _pub_fn_signatures(_module(src, mod)).items():
            ours[f"{mod}::{name}"] = sig
    for name, want in REFERENCE_SIGNATURES.items():
        assert ours.get(name) == want, f"{name}: crate has {ours.get(name)!r}, the reference {want!r}"


def test_reference_signature_table_matches_the_reference_text():
    """Only where the reference's sources are at hand (they do not travel with the repository)."""
    import pytest

    ref = "/root/reference/src"
    if not os.path.isdir(ref):
        pytest.skip("reference sources not present on this machine")
    for mod in ("quant", "gguf"):
        theirs = _pub_fn_signatures(open(os.path.join(ref, f"{mod}.rs")).read())
        for name, want in REFERENCE_SIGNATURES.items():
            if name.startswith(mod + "::"):
                assert theirs.get(name.split("::")[1]) == want, f"{name}: reference has {theirs.get(name.split('::')[1])!r}"
