#!/usr/bin/env python3
"""Writes src/lib.rs from include/autograph_hip.h: one `pub fn` per entry point, in header order,
with the C types mapped to their Rust FFI equivalents.  Run it after the header changes:

    python3 rust/autograph-hip-sys/gen_bindings.py
"""
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "..", "..", "include", "autograph_hip.h")
OUT = os.path.join(HERE, "src", "lib.rs")

SCALARS = {"int": "c_int", "int64_t": "i64", "float": "f32", "size_t": "usize", "char": "c_char", "void": "c_void"}

PREAMBLE = '''//! Raw bindings to `libautograph_hip.so` (the C ABI of `include/autograph_hip.h`), one declaration
//! per entry point, in header order.  Status codes: 0 ok, negative argument errors (`AGH_E*`),
//! positive `hipError_t`.  This crate is source only: it has not been compiled (the image it was
//! written in has no Rust toolchain); `gen_bindings.py` writes this file from the header and
//! `tests/test_abi_cpu.py` checks every argument type against the header.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};
'''


def rust_type(ctype):
    """`const void *` -> `*const c_void`, `void **` -> `*mut *mut c_void`, `int64_t` -> `i64`."""
    toks = ctype.replace("*", " * ").split()
    const = "const" in toks
    toks = [t for t in toks if t != "const"]
    base, stars = toks[0], toks.count("*")
    out = SCALARS[base]
    for level in range(stars):
        out = ("*const " if const and level == 0 else "*mut ") + out
    return out


def parse(header_text):
    text = re.sub(r"/\*.*?\*/", "", header_text, flags=re.S)
    consts = re.findall(r"#define\s+(AGH_[A-Z_0-9]+)\s+\(?(-?\d+)\)?", text)
    decls = []
    for ret, name, args in re.findall(r"^\s*([a-z_0-9 ]+?\s*\**)\s*\b(agh_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text, flags=re.M):
        params = []
        if args.strip() not in ("", "void"):
            for a in args.split(","):
                m = re.match(r"\s*(.*?)([A-Za-z_][A-Za-z_0-9]*)\s*$", a.replace("\n", " "))
                params.append((m.group(2), rust_type(m.group(1))))
        decls.append((name, params, rust_type(ret)))
    return consts, decls


def render(consts, decls):
    lines = [PREAMBLE]
    for name, value in consts:
        if name == "AGH_NOALLOC_SCRATCH_BYTES":
            lines.append(f"pub const {name}: usize = {value};")
        else:
            lines.append(f"pub const {name}: c_int = {value};")
    lines.append("")
    lines.append('#[link(name = "autograph_hip")]')
    lines.append('extern "C" {')
    for name, params, ret in decls:
        args = ", ".join(f"{n}: {t}" for n, t in params)
        lines.append(f"    pub fn {name}({args}) -> {ret};")
    lines.append("}")
    return "\n".join(lines) + "\n"


if __name__ == "__main__":
    consts, decls = parse(open(HEADER).read())
    open(OUT, "w").write(render(consts, decls))
    print(f"{OUT}: {len(decls)} entry points")
