#!/usr/bin/env python3
"""Writes src/lib.rs of the rllama-hip-sys crate from include/rllama_hip.h.

    python rust/rllama-hip-sys/gen_bindings.py [--check]

The crate is the `extern "C"` seam a Rust host (rllama with a `hip` feature in the place of `opencl`, Cargo.toml:42-44 of
the reference) links against.  Every function, enum value and struct of the header appears once; --check exits non-zero
when src/lib.rs is not what the header produces (tests/test_abi.py runs the same comparison).
"""
from __future__ import annotations

import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "..", "..", "include", "rllama_hip.h")
OUT = os.path.join(HERE, "src", "lib.rs")

OPAQUE = ("rlh_ctx", "rlh_model", "rlh_caches", "rlh_tensor", "rlh_event")
SCALARS = {"int": "c_int", "float": "c_float", "double": "c_double", "char": "c_char", "void": "c_void", "int32_t": "i32",
           "uint16_t": "u16", "uint64_t": "u64", "size_t": "usize"}


def strip_comments(text: str) -> str:
    return re.sub(r"/\*.*?\*/", "", text, flags=re.S)


def rust_type(ctype: str) -> str:
    """'const rlh_model_params *' -> '*const rlh_model_params', 'rlh_ctx **' -> '*mut *mut rlh_ctx', 'int' -> 'c_int'."""
    t = ctype.strip()
    stars = t.count("*")
    base = t.replace("*", " ").split()
    const = "const" in base
    base = [b for b in base if b not in ("const", "struct")]
    assert len(base) == 1, ctype
    name = SCALARS.get(base[0], base[0])
    out = name
    for i in range(stars):
        # in C the `const` of these declarations always qualifies the pointee of the innermost pointer
        out = ("*const " if (const and i == 0) else "*mut ") + out
    return out


def parse(text: str):
    text = strip_comments(text)
    funcs = []
    for m in re.finditer(r"(?m)^(const char \*|int|void)\s*(rlh_[a-z0-9_]+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        ret, name, args = m.group(1).strip(), m.group(2), " ".join(m.group(3).split())
        params = []
        if args != "void":
            for a in args.split(","):
                a = a.strip()
                pm = re.match(r"^(.*?)([A-Za-z_][A-Za-z0-9_]*)$", a)
                params.append((pm.group(2), rust_type(pm.group(1))))
        rret = {"int": "c_int", "void": None, "const char *": "*const c_char"}[ret]
        funcs.append((name, params, rret))
    enums = []
    for m in re.finditer(r"typedef enum\s*\{(.*?)\}\s*(rlh_[a-z_]+)\s*;", text, flags=re.S):
        items = []
        for it in m.group(1).split(","):
            it = it.strip()
            if it:
                k, v = it.split("=")
                items.append((k.strip(), int(v.strip())))
        enums.append((m.group(2), items))
    structs = []
    for m in re.finditer(r"typedef struct(?:\s+rlh_[a-z_]+)?\s*\{(.*?)\}\s*(rlh_[a-z_]+)\s*;", text, flags=re.S):
        fields = []
        for f in m.group(1).split(";"):
            f = " ".join(f.split())
            if f:
                fm = re.match(r"^(.*?)([A-Za-z_][A-Za-z0-9_]*)$", f)
                fields.append((fm.group(2), rust_type(fm.group(1))))
        structs.append((m.group(2), fields))
    version = int(re.search(r"#define RLH_ABI_VERSION (\d+)", text).group(1))
    return funcs, enums, structs, version


RUST_KEYWORDS = {"type", "ref", "in", "box", "fn", "mod", "move", "match", "loop", "impl", "use", "where", "self", "super"}


def render(funcs, enums, structs, version) -> str:
    o = []
    o.append("//! Raw bindings to `librllama_hip.so`: rllama's per-token transformer forward path on one MI355X (gfx950).")
    o.append("//!")
    o.append("//! GENERATED from `include/rllama_hip.h` by `gen_bindings.py`; edit the header and run the generator, not this file.")
    o.append("//! The header's comments say what each call replaces in rllama (`OpenCL`, `OpenCLTensor`, `Transformer::forward`, ...).")
    o.append("#![allow(non_camel_case_types, non_snake_case)]")
    o.append("")
    o.append("use std::os::raw::{c_char, c_double, c_float, c_int, c_void};")
    o.append("")
    o.append(f"pub const RLH_ABI_VERSION: c_int = {version};")
    o.append("")
    for name in OPAQUE:
        o.append("#[repr(C)]")
        o.append(f"pub struct {name} {{")
        o.append("    _private: [u8; 0],")
        o.append("}")
    o.append("")
    for ename, items in enums:
        o.append(f"// {ename}")
        for k, v in items:
            o.append(f"pub const {k}: c_int = {v};")
        o.append("")
    for sname, fields in structs:
        o.append("#[repr(C)]")
        o.append("#[derive(Clone, Copy, Debug)]")
        o.append(f"pub struct {sname} {{")
        for fname, ftype in fields:
            o.append(f"    pub {fname}: {ftype},")
        o.append("}")
        o.append("")
    o.append('#[link(name = "rllama_hip")]')
    o.append('extern "C" {')
    for name, params, ret in funcs:
        ps = ", ".join(f"{('r#' + p) if p in RUST_KEYWORDS else p}: {t}" for p, t in params)
        o.append(f"    pub fn {name}({ps}){' -> ' + ret if ret else ''};")
    o.append("}")
    o.append("")
    return "\n".join(o)


def generate() -> str:
    return render(*parse(open(HEADER).read()))


def main() -> int:
    text = generate()
    if "--check" in sys.argv:
        cur = open(OUT).read() if os.path.exists(OUT) else ""
        if cur != text:
            print("rust/rllama-hip-sys/src/lib.rs is out of date with include/rllama_hip.h", file=sys.stderr)
            return 1
        return 0
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    with open(OUT, "w") as f:
        f.write(text)
    print(f"wrote {OUT}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
