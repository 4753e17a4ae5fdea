#!/usr/bin/env python3
"""Prints a Rust ``-sys`` module (``extern "C"`` declarations, ``#[repr(C)]`` structs and the
constants) generated from mxp.h, for a Rust caller of libmxplace.so:

    python include/gen_rust_sys.py > mxplace-sys/src/lib.rs

The header is the single source of truth; this keeps a Rust binding from drifting.  Only the
C subset mxp.h uses is understood (fixed-width integers, double, char, void, pointers to
those and to the header's own structs, fixed-size arrays inside structs, object-like
``#define`` constants).
"""

from __future__ import annotations

import re
import sys
from pathlib import Path

HEADER = Path(__file__).with_name("mxp.h")

SCALARS = {"int": "c_int", "int32_t": "i32", "int64_t": "i64", "uint8_t": "u8", "uint16_t": "u16", "uint32_t": "u32",
           "uint64_t": "u64", "double": "f64", "float": "f32", "char": "c_char", "void": "c_void", "size_t": "usize"}


def strip_comments(text: str) -> str:
    return re.sub(r"/\*.*?\*/", "", text, flags=re.S)


def rust_type(ctype: str, structs: set) -> str:
    """``const void* const*`` -> ``*const *const c_void`` and so on."""
    t = ctype.strip()
    if "*" not in t:
        base = t.replace("const", "").strip()
        if base in SCALARS:
            return SCALARS[base]
        if base in structs:
            return base
        raise ValueError(f"unknown C type '{ctype}'")
    head, _star, tail = t.rpartition("*")
    inner = rust_type(head, structs) if "*" in head else None
    pointee_const = "const" in (head.split("*")[-1] if "*" in head else head)
    if inner is None:
        base = head.replace("const", "").strip()
        inner = SCALARS.get(base, base if base in structs else None)
        if inner is None:
            raise ValueError(f"unknown C type '{ctype}'")
    # qualifiers written after the last '*' (``* const``) bind to the pointer itself: irrelevant in Rust
    _ = tail
    return ("*const " if pointee_const else "*mut ") + inner


def parse(text: str):
    text = strip_comments(text)
    consts = []
    for m in re.finditer(r"^#define[ \t]+(MXP_[A-Z0-9_]+)[ \t]+([^\n]+?)[ \t]*$", text, flags=re.M):
        name, val = m.group(1), m.group(2).strip()
        if name.endswith("_H") or "(" in val and not re.fullmatch(r"\(?-?[0-9xa-fA-Fu]+\)?", val):
            continue
        consts.append((name, val))
    opaque = re.findall(r"typedef\s+struct\s+(\w+)\s+\1\s*;", text)
    structs = {}
    for m in re.finditer(r"typedef\s+struct\s+(\w+)\s*\{(.*?)\}\s*\1\s*;", text, flags=re.S):
        fields = []
        for decl in m.group(2).split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            fm = re.fullmatch(r"(.+?[\s\*])(\w+)(\[(\w+)\])?", decl)
            fields.append((fm.group(1).strip(), fm.group(2), fm.group(4)))
        structs[m.group(1)] = fields
    funcs = []
    body = re.sub(r"typedef\s+struct\s+\w+\s*\{.*?\}\s*\w+\s*;", "", text, flags=re.S)
    for m in re.finditer(r"^([\w\s\*]+?[\s\*])(mxp_\w+)\s*\(([^;{}]*?)\)\s*;", body, flags=re.M | re.S):
        ret, name, args = " ".join(m.group(1).split()), m.group(2), " ".join(m.group(3).split())
        params = []
        if args and args != "void":
            for a in args.split(","):
                a = a.strip()
                arr = re.fullmatch(r"(.+?[\s\*])(\w+)\[\w*\]", a)  # an array parameter is a pointer
                if arr:
                    params.append((arr.group(1).strip() + "*", arr.group(2)))
                    continue
                am = re.fullmatch(r"(.+?[\s\*])(\w+)", a)
                params.append((am.group(1).strip(), am.group(2)))
        funcs.append((ret, name, params))
    return consts, opaque, structs, funcs


def const_value(val: str, names: dict) -> tuple[str, str]:
    v = val.strip("()")
    if v in names:
        return names[v]
    ty = "u32" if v.lower().endswith("u") else "i32"
    return ty, v.rstrip("uU")


def generate(text: str) -> str:
    consts, opaque, structs, funcs = parse(text)
    names = set(opaque) | set(structs)
    out = ["// Generated from mxp.h by gen_rust_sys.py; do not edit.", "#![allow(non_camel_case_types)]", "",
           "use std::os::raw::{c_char, c_int, c_void};", ""]
    seen = {}
    for name, val in consts:
        ty, v = const_value(val, seen)
        seen[name] = (ty, v)
        out.append(f"pub const {name}: {ty} = {v};")
    out.append("")
    for o in opaque:
        out += ["#[repr(C)]", f"pub struct {o} {{ _private: [u8; 0] }}", ""]
    for sname, fields in structs.items():
        out += ["#[repr(C)]", "#[derive(Clone, Copy)]", f"pub struct {sname} {{"]
        for ctype, fname, dim in fields:
            rt = rust_type(ctype, names)
            if dim:
                rt = f"[{rt}; {dim} as usize]" if not dim.isdigit() else f"[{rt}; {dim}]"
            out.append(f"    pub {fname}: {rt},")
        out += ["}", ""]
    out += ['#[link(name = "mxplace")]', 'extern "C" {']
    for ret, name, params in funcs:
        args = ", ".join(f"{'type_' if p == 'type' else p}: {rust_type(t, names)}" for t, p in params)
        r = "" if ret == "void" else f" -> {rust_type(ret, names)}"
        out.append(f"    pub fn {name}({args}){r};")
    out += ["}", ""]
    return "\n".join(out)


if __name__ == "__main__":
    sys.stdout.write(generate(HEADER.read_text()))
