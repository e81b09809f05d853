#!/usr/bin/env python3
"""Writes src/ffi.rs from include/ojas_mi355x.h: one `extern "C"` declaration per entry point, the
`#[repr(C)]` structs and the status / dtype constants. Run it again whenever the header changes:

    python3 ojas-mi355x/gen_ffi.py            # rewrites ojas-mi355x/src/ffi.rs
    python3 ojas-mi355x/gen_ffi.py --check    # exits 1 if src/ffi.rs is out of date
"""
import re
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent
HEADER = ROOT.parent / "include" / "ojas_mi355x.h"
OUT = ROOT / "src" / "ffi.rs"

SCALARS = {"int32_t": "i32", "uint32_t": "u32", "int64_t": "i64", "uint64_t": "u64", "float": "f32", "double": "f64",
           "size_t": "usize", "char": "c_char", "void": "c_void", "unsigned long long": "u64", "int": "c_int"}


def rust_name(c_name: str) -> str:
    """omx_adamw_config -> OmxAdamwConfig."""
    return "".join(part.capitalize() for part in c_name.split("_"))


def strip_comments(text: str) -> str:
    return re.sub(r"/\*.*?\*/", "", text, flags=re.S)


def rust_type(c_type: str, structs) -> str:
    """A C parameter or field type -> Rust. Pointers keep their constness level by level."""
    t = " ".join(c_type.replace("*", " * ").split())
    tokens = t.split(" ")
    base, i = [], 0
    while i < len(tokens) and tokens[i] != "*":
        base.append(tokens[i])
        i += 1
    const = "const" in base
    base = " ".join(b for b in base if b not in ("const", "struct"))
    if base in SCALARS:
        rust = SCALARS[base]
    elif base in structs:
        rust = rust_name(base)
    else:
        raise ValueError(f"unknown C type {c_type!r}")
    # each '*' wraps what came before it; a 'const' right after a '*' makes the NEXT level const
    while i < len(tokens):
        assert tokens[i] == "*", c_type
        rust = ("*const " if const else "*mut ") + rust
        const = i + 1 < len(tokens) and tokens[i + 1] == "const"
        i += 2 if const else 1
    return rust


def parse(text: str):
    text = strip_comments(text)
    structs, order = {}, []
    for m in re.finditer(r"typedef\s+struct\s*(\w*)\s*\{(.*?)\}\s*(\w+)\s*;", text, re.S):
        fields = []
        for decl in m.group(2).split(";"):
            decl = decl.strip()
            if not decl:
                continue
            c_type, names = re.match(r"(.*?[\s\*])(\w+(?:\s*,\s*\w+)*)$", decl, re.S).groups()
            for n in names.split(","):
                fields.append((n.strip(), c_type.strip()))
        structs[m.group(3)] = fields
        order.append(m.group(3))
    opaque = re.findall(r"typedef\s+struct\s+(\w+)\s+(\w+)\s*;", text)
    for _, name in opaque:
        structs.setdefault(name, None)
    enums = []
    for m in re.finditer(r"(?:typedef\s+)?enum\s*\w*\s*\{(.*?)\}\s*(\w*)\s*;", text, re.S):
        value = -1
        for item in m.group(1).split(","):
            item = item.strip()
            if not item:
                continue
            if "=" in item:
                name, v = (s.strip() for s in item.split("="))
                value = int(v, 0)
            else:
                name, value = item, value + 1
            enums.append((name, value))
    functions = []
    for m in re.finditer(r"\n\s*([\w\s\*]+?)\b(omx_\w+)\s*\(([^;{]*?)\)\s*;", text, re.S):
        ret, name, params = m.group(1).strip(), m.group(2), m.group(3)
        args = []
        if params.strip() and params.strip() != "void":
            for p in params.split(","):
                c_type, pname = re.match(r"(.*?[\s\*])(\w+)$", p.strip(), re.S).groups()
                args.append((pname, c_type.strip()))
        functions.append((name, ret, args))
    return structs, order, opaque, enums, functions


KEYWORDS = {"type", "in", "ref", "move", "box", "loop", "match", "mod", "priv", "self", "use", "where"}


def render() -> str:
    structs, order, opaque, enums, functions = parse(HEADER.read_text())
    out = ["//! `extern \"C\"` declarations for `libojas_mi355x.so`: one per entry point of include/ojas_mi355x.h.",
           "//! Written by gen_ffi.py from that header; edit the header and run the script, not this file.",
           "#![allow(non_camel_case_types, clippy::too_many_arguments)]", "",
           "use std::os::raw::{c_char, c_int, c_void};", ""]
    for _, name in opaque:
        out += ["#[repr(C)]", f"pub struct {rust_name(name)} {{", "    _private: [u8; 0],", "}", ""]
    for name in order:
        out += ["#[repr(C)]", "#[derive(Clone, Copy, Debug)]", f"pub struct {rust_name(name)} {{"]
        out += [f"    pub {f}: {rust_type(t, structs)}," for f, t in structs[name]]
        out += ["}", ""]
    for name, value in enums:
        out.append(f"pub const {name}: i32 = {value};")
    out += ["", "extern \"C\" {"]
    for name, ret, args in functions:
        params = ", ".join(f"{('r#' + a) if a in KEYWORDS else a}: {rust_type(t, structs)}" for a, t in args)
        tail = "" if ret == "void" else f" -> {rust_type(ret, structs)}"
        out.append(f"    pub fn {name}({params}){tail};")
    out += ["}", ""]
    return "\n".join(out)


def main() -> int:
    text = render()
    if "--check" in sys.argv:
        if not OUT.exists() or OUT.read_text() != text:
            print(f"{OUT} is out of date: run {Path(__file__).name}", file=sys.stderr)
            return 1
        return 0
    OUT.write_text(text)
    print(f"wrote {OUT} ({text.count('pub fn ')} functions)")
    return 0


if __name__ == "__main__":
    sys.exit(main())
