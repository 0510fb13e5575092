#!/usr/bin/env python3
"""Writes src/lib.rs of the cutile-hip-sys crate from include/cutile_hip.h.

    python rust/cutile-hip-sys/gen_bindings.py            # rewrites rust/cutile-hip-sys/src/lib.rs
    python rust/cutile-hip-sys/gen_bindings.py --check    # exit 1 if src/lib.rs is not what the header gives

The header is plain C99 of a narrow shape (typedefs of handles, anonymous and named enums, records of fixed-width
fields, function-pointer typedefs, one prototype per export), so a small declaration reader is enough; no C compiler
and no bindgen is involved.  tests/test_rust_bindings.py reads the header and the generated file with a reader of its
own and compares them declaration by declaration.
"""
from __future__ import annotations

import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "..", "..", "include", "cutile_hip.h")
OUT = os.path.join(HERE, "src", "lib.rs")

SCALARS = {
    "int32_t": "i32", "uint32_t": "u32", "int64_t": "i64", "uint64_t": "u64", "uint8_t": "u8", "int8_t": "i8",
    "uint16_t": "u16", "int16_t": "i16", "size_t": "usize", "float": "f32", "double": "f64", "char": "c_char",
    "unsigned char": "u8", "void": "c_void", "int": "c_int", "unsigned": "c_uint", "unsigned int": "c_uint",
}


def strip_comments(text: str) -> str:
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def rust_type(c: str, known: set[str]) -> str:
    """C type text (no declarator name) -> Rust type"""
    c = " ".join(c.replace("*", " * ").split())
    toks = c.split(" ")
    # read left to right: [const] base {* [const]}
    i = 0
    const_base = False
    if toks[i] == "const":
        const_base = True
        i += 1
    base = toks[i]
    i += 1
    if base == "unsigned" and i < len(toks) and toks[i] in ("char", "int"):
        base += " " + toks[i]
        i += 1
    if i < len(toks) and toks[i] == "const":      # "char const"
        const_base = True
        i += 1
    if base in SCALARS:
        ty = SCALARS[base]
    elif base in known:
        ty = base
    else:
        raise ValueError(f"unknown C type {base!r} in {c!r}")
    pointee_const = const_base
    while i < len(toks):
        if toks[i] != "*":
            raise ValueError(f"cannot read {c!r}")
        ty = ("*const " if pointee_const else "*mut ") + ty
        pointee_const = False
        i += 1
        if i < len(toks) and toks[i] == "const":
            pointee_const = True
            i += 1
    if base == "void" and not ty.startswith("*"):
        return "()"
    return ty


def split_declarator(decl: str):
    """'const uint32_t grid[3]' -> ('const uint32_t', 'grid', '3'); 'void* user' -> ('void*', 'user', None)"""
    decl = decl.strip()
    m = re.match(r"^(.*?)(\b[A-Za-z_]\w*)\s*(?:\[\s*(\w*)\s*\])?$", decl, flags=re.S)
    if not m:
        raise ValueError(f"cannot read declarator {decl!r}")
    ty, name, dim = m.group(1).strip(), m.group(2), m.group(3)
    if not ty:      # unnamed parameter: the "name" was the type
        return decl, None, None
    return ty, name, dim


def read_header(text: str):
    text = strip_comments(text)
    text = re.sub(r"^\s*#\s*(ifdef|ifndef|endif|include|if|else)\b[^\n]*", "", text, flags=re.M)
    text = text.replace('extern "C" {', "")
    defines = [(m.group(1), m.group(2)) for m in re.finditer(r"^\s*#\s*define\s+(\w+)\s+(-?\w+)\s*$", text, flags=re.M)]
    text = re.sub(r"^\s*#\s*define[^\n]*", "", text, flags=re.M)
    items = []          # in header order: (kind, payload)
    known: set[str] = set()
    pos = 0
    # statements end at ';' outside braces
    depth, start = 0, 0
    stmts = []
    for i, ch in enumerate(text):
        if ch == "{":
            depth += 1
        elif ch == "}":
            depth -= 1
            if depth < 0:      # the closing brace of extern "C"
                depth = 0
                start = i + 1
        elif ch == ";" and depth == 0:
            stmts.append(" ".join(text[start:i].split()))
            start = i + 1
    for st in stmts:
        if not st:
            continue
        m = re.match(r"^typedef struct (\w+)\s*\* (\w+)$", st) or re.match(r"^typedef struct (\w+)\s*\*\s*(\w+)$", st)
        if m:
            items.append(("opaque", (m.group(1), m.group(2))))
            known.add(m.group(2))
            continue
        m = re.match(r"^typedef struct \{(.*)\} (\w+)$", st)
        if m:
            fields = []
            for f in m.group(1).split(";"):
                f = f.strip()
                if not f:
                    continue
                first, *rest = [p.strip() for p in f.split(",")]
                ty, name, dim = split_declarator(first)
                fields.append((ty, name, dim))
                for r in rest:
                    rm = re.match(r"^(\w+)(?:\[(\w+)\])?$", r)
                    fields.append((ty, rm.group(1), rm.group(2)))
            items.append(("struct", (m.group(2), fields)))
            known.add(m.group(2))
            continue
        m = re.match(r"^(typedef )?enum \{(.*)\}\s*(\w+)?$", st)
        if m:
            consts, nxt = [], 0
            for e in m.group(2).split(","):
                e = e.strip()
                if not e:
                    continue
                if "=" in e:
                    n, v = [p.strip() for p in e.split("=")]
                    nxt = int(v, 0)
                else:
                    n = e
                consts.append((n, nxt))
                nxt += 1
            items.append(("enum", (m.group(3), consts)))
            if m.group(3):
                known.add(m.group(3))
            continue
        m = re.match(r"^typedef (.*?)\(\s*\*\s*(\w+)\s*\)\s*\((.*)\)$", st)
        if m:
            params = [] if m.group(3).strip() == "void" else [split_declarator(p) for p in m.group(3).split(",")]
            items.append(("fnptr", (m.group(2), m.group(1).strip(), params)))
            known.add(m.group(2))
            continue
        m = re.match(r"^typedef (.*\S)\s+(\w+)$", st) or re.match(r"^typedef (.*\*)\s*(\w+)$", st)
        if m:
            items.append(("alias", (m.group(2), m.group(1).strip())))
            known.add(m.group(2))
            continue
        m = re.match(r"^(.*?)\b(\w+)\s*\((.*)\)$", st)
        if m:
            params = [] if m.group(3).strip() == "void" else [split_declarator(p) for p in m.group(3).split(",")]
            items.append(("fn", (m.group(2), m.group(1).strip(), params)))
            continue
        raise ValueError(f"unread statement: {st!r}")
    return defines, items, known


def param_type(ty: str, dim, known) -> str:
    if dim is not None:      # an array parameter is a pointer to its element
        return rust_type(ty + " *", known)
    return rust_type(ty, known)


def render(defines, items, known) -> str:
    out = []
    w = out.append
    w("//! Raw FFI declarations of `libcutile_hip.so` — one item per declaration of `include/cutile_hip.h`, in the")
    w("//! header's order.  This is the crate that takes the place of `cuda-bindings` / the driver half of `cuda-core`")
    w("//! (cuda-bindings/src/lib.rs:16, cuda-core/src/cudarc_shim.rs:28-807) under the reference's host crates.")
    w("//!")
    w("//! GENERATED by `gen_bindings.py` from the header; do not edit.  NOT COMPILED in the environment this was")
    w("//! written in (it has no Rust toolchain): `tests/test_rust_bindings.py` compares every declaration here with")
    w("//! the header instead (names, argument count, pointer / integer / float class and width per position, record")
    w("//! field order and sizes, constant values).")
    w("#![allow(non_camel_case_types, non_upper_case_globals, unused_imports)]")
    w("#![no_std]")
    w("")
    w("use core::ffi::{c_char, c_int, c_uint, c_void};")
    w("")
    for name, val in defines:
        if name.endswith("_H"):
            continue
        ty = "usize" if name == "CUTILE_MAX_RANK" else "i32"
        w(f"pub const {name}: {ty} = {val};")
    w("")
    fns = []
    for kind, p in items:
        if kind == "opaque":
            tag, alias = p
            w("#[repr(C)]")
            w(f"pub struct {tag} {{")
            w("    _private: [u8; 0],")
            w("}")
            w(f"pub type {alias} = *mut {tag};")
        elif kind == "alias":
            name, cty = p
            w(f"pub type {name} = {rust_type(cty, known)};")
        elif kind == "enum":
            name, consts = p
            if name:
                w(f"pub type {name} = c_int;")
            for n, v in consts:
                w(f"pub const {n}: {name or 'i32'} = {v};")
        elif kind == "struct":
            name, fields = p
            w("#[repr(C)]")
            w("#[derive(Clone, Copy)]")
            w(f"pub struct {name} {{")
            for ty, fname, dim in fields:
                rt = rust_type(ty, known)
                if dim is not None:
                    rt = f"[{rt}; {dim}]"
                w(f"    pub {fname}: {rt},")
            w("}")
        elif kind == "fnptr":
            name, ret, params = p
            args = ", ".join(f"{pn or 'arg'}: {param_type(ty, dim, known)}" for ty, pn, dim in params)
            r = rust_type(ret, known)
            w(f"pub type {name} = Option<unsafe extern \"C\" fn({args}){'' if r == '()' else ' -> ' + r}>;")
        elif kind == "fn":
            fns.append(p)
            continue
        w("")
    w('#[link(name = "cutile_hip")]')
    w('extern "C" {')
    for name, ret, params in fns:
        args = ", ".join(f"{('r#' + pn) if pn in ('fn', 'type', 'ref', 'in', 'box', 'loop', 'match', 'move', 'mod', 'use', 'where') else (pn or 'arg')}: "
                         f"{param_type(ty, dim, known)}" for ty, pn, dim in params)
        r = rust_type(ret, known)
        w(f"    pub fn {name}({args}){'' if r == '()' else ' -> ' + r};")
    w("}")
    return "\n".join(out) + "\n"


def generate() -> str:
    with open(HEADER) as f:
        defines, items, known = read_header(f.read())
    return render(defines, items, known)


if __name__ == "__main__":
    text = generate()
    if "--check" in sys.argv:
        cur = open(OUT).read() if os.path.exists(OUT) else ""
        sys.exit(0 if cur == text else "rust/cutile-hip-sys/src/lib.rs is stale: run rust/cutile-hip-sys/gen_bindings.py")
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    with open(OUT, "w") as f:
        f.write(text)
    print(OUT)
