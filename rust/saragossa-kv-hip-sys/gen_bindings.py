#!/usr/bin/env python3
"""Writes src/lib.rs, the raw Rust binding of include/saragossa_kv.h: one `pub fn` per C
prototype, one `pub const` per #define, one opaque struct per handle type. Run it again after
the header changes (tests/test_rust_sys_crate.py fails when the two are out of step):

    python3 rust/saragossa-kv-hip-sys/gen_bindings.py
"""
from __future__ import annotations

import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "..", "..", "include", "saragossa_kv.h")
OUT = os.path.join(HERE, "src", "lib.rs")

SCALARS = {"int32_t": "i32", "uint64_t": "u64", "uint32_t": "u32", "uint16_t": "u16", "uint8_t": "u8",
           "size_t": "usize", "float": "f32", "char": "c_char", "void": "c_void"}


def strip_comments(text: str) -> str:
    return re.sub(r"/\*.*?\*/", "", text, flags=re.S)


def rust_type(c: str, opaque: set) -> str:
    """A C parameter or return type (no name) as a Rust FFI type."""
    c = " ".join(c.replace("*", " * ").split())
    if c == "skv_stream":
        return "skv_stream"
    toks = c.split()
    # base type with an optional leading const
    const_base = toks[0] == "const"
    if const_base:
        toks = toks[1:]
    base = toks[0]
    rest = toks[1:]
    if base in SCALARS:
        r = SCALARS[base]
    elif base in opaque or base == "skv_hit":
        r = base
    else:
        raise ValueError("unknown C type: " + c)
    # each '*' adds a pointer level; a 'const' right after a '*' makes THAT pointer const, which
    # decides the mutability of the next level out
    inner_const = const_base
    i = 0
    while i < len(rest):
        if rest[i] != "*":
            raise ValueError("cannot parse: " + c)
        r = ("*const " if inner_const else "*mut ") + r
        inner_const = i + 1 < len(rest) and rest[i + 1] == "const"
        i += 2 if inner_const else 1
    if not rest and base == "void":
        return "()"
    return r


def split_args(args: str):
    args = args.strip()
    if args in ("", "void"):
        return []
    return [a.strip() for a in args.split(",")]


def parse_header(text: str):
    text = strip_comments(text)
    consts = re.findall(r"^#define\s+(SKV_[A-Z0-9_]+)\s+(.+?)\s*$", text, flags=re.M)
    opaque = set(re.findall(r"typedef\s+struct\s+(skv_[a-z_]+)\s+\1\s*;", text))
    body = re.sub(r"^#.*$", "", text, flags=re.M)
    body = re.sub(r"typedef\s+struct\s+skv_hit\s*\{.*?\}\s*skv_hit\s*;", "", body, flags=re.S)
    body = re.sub(r"typedef[^;]*;", "", body)
    body = body.replace('extern "C" {', "").replace("}", "")
    protos = []
    for stmt in body.split(";"):
        stmt = " ".join(stmt.split())
        if not stmt:
            continue
        m = re.match(r"^(.*?)\b(skv_[a-z0-9_]+)\s*\((.*)\)$", stmt)
        if not m:
            raise ValueError("not a prototype: " + stmt)
        ret, name, args = m.group(1).strip(), m.group(2), split_args(m.group(3))
        params = []
        for a in args:
            arr = re.match(r"^(.*?)(\w+)\s*\[\s*\d*\s*\]$", a)       # uint8_t out[32]
            if arr:
                ctype, pname = arr.group(1).strip() + " *", arr.group(2)
            else:
                pm = re.match(r"^(.*?)(\w+)$", a)
                ctype, pname = pm.group(1).strip(), pm.group(2)
            params.append((pname, rust_type(ctype, opaque)))
        protos.append((name, params, rust_type(ret, opaque)))
    return consts, sorted(opaque), protos


def const_value(v: str):
    m = re.match(r"^\(\(size_t\)\s*(\d+)\s*<<\s*(\d+)\)$", v)
    if m:
        return "usize", "%s << %s" % (m.group(1), m.group(2))
    if re.match(r"^-?\d+$", v):
        return "i32", v
    raise ValueError("cannot translate #define value: " + v)


def render(consts, opaque, protos) -> str:
    out = ["// Raw FFI binding of include/saragossa_kv.h (libsaragossa_kv.so, the gfx950 KV-cache hot path).",
           "// Written by gen_bindings.py from the header: one declaration per C prototype, nothing else.",
           "// No Rust toolchain exists where this file is produced: it has not been compiled there.",
           "#![allow(non_camel_case_types)]",
           "use std::os::raw::{c_char, c_void};",
           ""]
    for name in opaque:
        out.append("#[repr(C)] pub struct %s { _private: [u8; 0] }" % name)
    out += ["",
            "/// PrefixBlockHit with an opaque payload (src/serve/cache.rs:50-60).",
            "#[repr(C)]",
            "#[derive(Clone, Copy)]",
            "pub struct skv_hit { pub tokens: usize, pub hash: [u8; 32], pub payload: u64, pub matched_blocks: usize }",
            "",
            "/// A hipStream_t; null is the default stream.",
            "pub type skv_stream = *mut c_void;",
            ""]
    for name, value in consts:
        if name == "SARAGOSSA_KV_H":
            continue
        ty, v = const_value(value)
        if name in ("SKV_PAGE_ROWS",):
            ty = "usize"
        out.append("pub const %s: %s = %s;" % (name, ty, v))
    out += ["", "#[link(name = \"saragossa_kv\")]", "extern \"C\" {"]
    for name, params, ret in protos:
        args = ", ".join("%s: %s" % (("r#" + p if p in ("type", "ref", "in", "match") else p), t) for p, t in params)
        out.append("    pub fn %s(%s)%s;" % (name, args, "" if ret == "()" else " -> " + ret))
    out += ["}", ""]
    return "\n".join(out)


def generate() -> str:
    return render(*parse_header(open(HEADER).read()))


if __name__ == "__main__":
    text = generate()
    if "--check" in sys.argv:
        sys.exit(0 if open(OUT).read() == text else 1)
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    open(OUT, "w").write(text)
    print("wrote", os.path.relpath(OUT), "(%d functions)" % text.count("pub fn "))
