#!/usr/bin/env python3
"""Regenerates the `extern "C"` block of src/lib.rs from include/peregrine_hip.h.

    python ffi/peregrine-hip-sys/gen_bindings.py            # rewrite src/lib.rs in place
    python ffi/peregrine-hip-sys/gen_bindings.py --check    # exit 1 if src/lib.rs is out of date

There is no Rust toolchain in the build image, so nothing compiles the crate here; this script and
tests/test_ffi_crate.py are what keep it in step with the header: every declaration, in header
order, with the C types mapped mechanically (rules in `rust_type`).
"""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "..", "..", "include", "peregrine_hip.h")
LIB_RS = os.path.join(HERE, "src", "lib.rs")
BEGIN, END = "// ---- generated from include/peregrine_hip.h: begin ----", "// ---- generated: end ----"

SCALARS = {"int": "c_int", "float": "f32", "double": "f64", "size_t": "usize", "char": "c_char", "void": "c_void",
           "int8_t": "i8", "uint8_t": "u8", "int16_t": "i16", "uint16_t": "u16", "int32_t": "i32", "uint32_t": "u32",
           "int64_t": "i64", "uint64_t": "u64", "pg_status": "pg_status"}
RUST_KEYWORDS = {"type", "in", "ref", "box", "move", "fn", "mod", "use", "where", "match", "loop", "impl", "trait", "self", "as"}


def declarations(text=None):
    """[(return C type, name, [(C type, parameter name)])] for every function the header declares."""
    text = open(HEADER).read() if text is None else text
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    out = []
    for m in re.finditer(r"([A-Za-z_][A-Za-z0-9_ \*]*?)\b(pg_[a-z0-9_]+)\s*\(([^;{}]*)\)\s*;", text):
        ret, name, args = " ".join(m.group(1).split()), m.group(2), " ".join(m.group(3).split())
        if ret.startswith("typedef"):
            continue
        params = []
        if args and args != "void":
            for a in args.split(","):
                mm = re.match(r"(.*?)([A-Za-z_][A-Za-z0-9_]*)$", a.strip())
                params.append((" ".join(mm.group(1).split()), mm.group(2)))
        out.append((ret, name, params))
    return out


def opaque_types(text=None):
    text = open(HEADER).read() if text is None else text
    return re.findall(r"typedef struct (pg_[a-z0-9_]+) \1;", text)


def rust_type(c):
    """`const T *const *` and friends -> `*const *const T`: a pointer level is `*const` when the
    thing it points at is const-qualified, else `*mut`; scalars by the table above; opaque
    handles keep their names."""
    toks = re.findall(r"\*|[A-Za-z_][A-Za-z0-9_]*", c)
    base, base_const, levels = None, False, []  # levels: constness of each pointer, innermost first
    for t in toks:
        if t == "const":
            if levels:
                levels[-1] = True
            else:
                base_const = True
        elif t == "*":
            levels.append(False)
        elif t in ("struct", "unsigned"):
            raise ValueError(f"unsupported C type {c!r}")
        else:
            base = t
    r = SCALARS.get(base, base)
    pointee_const = base_const
    for lvl_const in levels:
        r = ("*const " if pointee_const else "*mut ") + r
        pointee_const = lvl_const
    if not levels and base == "void":
        return ""
    return r


def rust_decl(ret, name, params):
    args = ", ".join(f"{(p + '_') if p in RUST_KEYWORDS else p}: {rust_type(t)}" for t, p in params)
    r = rust_type(ret)
    return f"    pub fn {name}({args})" + (f" -> {r};" if r else ";")


def generated_block():
    lines = [BEGIN, 'extern "C" {']
    lines += [rust_decl(*d) for d in declarations()]
    lines += ["}", END]
    return "\n".join(lines)


def main():
    src = open(LIB_RS).read()
    a, b = src.index(BEGIN), src.index(END) + len(END)
    new = src[:a] + generated_block() + src[b:]
    if "--check" in sys.argv:
        sys.exit(0 if new == src else "src/lib.rs is out of date: run gen_bindings.py")
    open(LIB_RS, "w").write(new)


if __name__ == "__main__":
    main()
