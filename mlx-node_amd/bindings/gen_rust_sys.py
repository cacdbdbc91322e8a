#!/usr/bin/env python3
"""Writes mxopt_sys.rs, the `extern "C"` half of a Rust `mxopt-sys` crate, from the three public headers:
every struct as #[repr(C)], every enum constant and #define as a const, every function as a declaration.
The headers are written in a small regular subset of C (one declaration per statement, no function
pointers, no unions, no bit-fields), which is all this reads.

    python mlx-node_amd/bindings/gen_rust_sys.py            rewrites mlx-node_amd/bindings/mxopt_sys.rs
    python mlx-node_amd/bindings/gen_rust_sys.py --check    exits 1 if the committed file is out of date

Nothing here was compiled (the build image has no Rust toolchain): the file is what a maintainer starts from.
"""
from __future__ import annotations

import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
# mxopt_diagnostics.h (probes, data generator, the pool scan on synthetic rates) is for benchmarks and tests only:
# no call site of the reference binds it, so it gets no Rust declarations.
HEADERS = ["mxopt.h", "mxopt_optimizers.h", "mxopt_engine.h"]
OUT = os.path.join(HERE, "mxopt_sys.rs")

SCALARS = {
    "void": "c_void", "char": "c_char", "int": "c_int", "float": "f32", "double": "f64", "size_t": "usize",
    "uint8_t": "u8", "uint32_t": "u32", "int32_t": "i32", "uint64_t": "u64", "int64_t": "i64", "ptrdiff_t": "isize",
}
RUST_KEYWORDS = {"type", "ref", "in", "fn", "loop", "match", "move", "mod", "use", "where", "self", "box"}


def strip_comments(text: str) -> str:
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def rust_type(ctype: str, opaque: set, structs: set) -> str:
    """`const char* const*` -> `*const *const c_char`, `mxopt_ctx**` -> `*mut *mut mxopt_ctx`, ..."""
    t = ctype.replace("struct ", "").strip()
    stars = []
    # peel pointers from the right: each '*' may be preceded by 'const' (pointee constness) and followed by 'const'
    while True:
        t = t.strip()
        if t.endswith("const") and "*" in t:
            t = t[:-5].strip()          # constness of the pointer variable itself: irrelevant in Rust
            continue
        if t.endswith("*"):
            t = t[:-1].strip()
            stars.append(None)
            continue
        break
    base_const = False
    words = t.split()
    if "const" in words:
        base_const = True
        words = [w for w in words if w != "const"]
    base = " ".join(words)
    if base == "unsigned long long":
        rbase = "u64"
    elif base in SCALARS:
        rbase = SCALARS[base]
    elif base in opaque or base in structs:
        rbase = base
    else:
        raise ValueError(f"unknown C type {ctype!r}")
    if not stars:
        return rbase
    # constness: the innermost pointer follows the base's const; outer ones follow the `const` written after the
    # star they point at -- the headers only ever write `const T*`, `T*`, `const T* const*`, `T**`.
    inner = "*const " if base_const else "*mut "
    out = inner + rbase
    for _ in stars[1:]:
        outer_const = bool(re.search(r"\*\s*const\s*\*", ctype))
        out = ("*const " if outer_const else "*mut ") + out
    return out


def ident(name: str) -> str:
    return "r#" + name if name in RUST_KEYWORDS else name


def parse(text: str):
    opaque = set(re.findall(r"typedef\s+struct\s+(\w+)\s+\1\s*;", text))
    structs, consts, functions = [], [], []
    for m in re.finditer(r"typedef\s+struct\s+(\w+)\s*\{(.*?)\}\s*\1\s*;", text, flags=re.S):
        fields = []
        for decl in m.group(2).split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            # `float bc1, bc2`, `const void* p` and `uint64_t per_region[MXOPT_N]`
            mm = re.match(r"(.+?[\s\*])([\w\s,\[\]]+)$", decl)
            ctype, names = mm.group(1).strip(), [n.strip() for n in mm.group(2).split(",")]
            for n in names:
                fields.append((ctype, n))
        structs.append((m.group(1), fields))
        opaque.discard(m.group(1))
    for m in re.finditer(r"#define\s+(MXOPT_[A-Z0-9_]+)\s+(0x[0-9a-fA-F]+u?|\d+u?)\b", text):
        consts.append((m.group(1), m.group(2).rstrip("u")))
    for m in re.finditer(r"enum\s*(?:\w+\s*)?\{(.*?)\}", text, flags=re.S):
        for entry in m.group(1).split(","):
            entry = " ".join(entry.split())
            if entry:
                name, value = [x.strip() for x in entry.split("=")]
                consts.append((name, value))
    body = re.sub(r"typedef\s+struct\s+\w+\s*\{.*?\}\s*\w+\s*;", "", text, flags=re.S)
    body = re.sub(r"enum\s*(?:\w+\s*)?\{.*?\}\s*;", "", body, flags=re.S)
    body = "\n".join(l for l in body.split("\n") if not l.lstrip().startswith("#") and 'extern "C"' not in l)
    body = re.sub(r"typedef\s+struct\s+\w+\s+\w+\s*;", "", body)
    for m in re.finditer(r"([\w\s\*]+?)\b(mxopt_\w+)\s*\(([^()]*)\)\s*;", body):
        ret = " ".join(m.group(1).split())
        if ret.startswith(("typedef", "#", "extern")) or not ret:
            continue
        params = []
        plist = " ".join(m.group(3).split())
        if plist and plist != "void":
            for p in plist.split(","):
                p = p.strip()
                mm = re.match(r"(.+?[\s\*])(\w+)$", p)
                params.append((mm.group(1).strip(), mm.group(2)))
        functions.append((ret, m.group(2), params))
    return opaque, structs, consts, functions


def generate() -> str:
    opaque, structs, consts, functions = set(), [], [], []
    per_header = []
    for h in HEADERS:
        text = strip_comments(open(os.path.join(ROOT, "include", h)).read())
        o, s, c, f = parse(text)
        opaque |= o
        per_header.append((h, s, c, f))
        structs += s
    struct_names = {n for n, _ in structs}
    opaque -= struct_names
    out = ["// Generated by mlx-node_amd/bindings/gen_rust_sys.py from include/mxopt.h, include/mxopt_optimizers.h and",
           "// include/mxopt_engine.h.  Do not edit: change the headers and regenerate.  The comments that say what",
           "// each entry point replaces in the reference are in the headers.",
           "#![allow(non_camel_case_types, non_upper_case_globals, dead_code)]",
           "use std::os::raw::{c_char, c_int, c_void};", ""]
    for name in sorted(opaque):
        out += ["#[repr(C)]", f"pub struct {name} {{ _private: [u8; 0] }}"]
    out.append("")
    seen_consts = set()
    for h, s, c, f in per_header:
        out.append(f"// ---- {h} " + "-" * max(4, 80 - len(h)))
        for cname, value in c:
            if cname in seen_consts or cname.endswith("_H"):
                continue
            seen_consts.add(cname)
            ctype = "u32" if cname.startswith("MXOPT_TF_") else "c_int"   # flag bits live in a uint32_t field
            out.append(f"pub const {cname}: {ctype} = {value};")
        if c:
            out.append("")
        for sname, fields in s:
            out += ["#[repr(C)]", "#[derive(Clone, Copy)]", f"pub struct {sname} {{"]
            for ctype, fname in fields:
                rt = rust_type(ctype, opaque, struct_names)
                arr = re.match(r"(\w+)\[(\w+)\]$", fname)
                if arr:     # fixed-size array member
                    fname, rt = arr.group(1), f"[{rt}; {arr.group(2)} as usize]"
                out.append(f"    pub {ident(fname)}: {rt},")
            out += ["}", ""]
        out.append('extern "C" {')
        for ret, fname, params in f:
            ps = ", ".join(f"{ident(n)}: {rust_type(t, opaque, struct_names)}" for t, n in params)
            r = "" if ret == "void" else f" -> {rust_type(ret, opaque, struct_names)}"
            out.append(f"    pub fn {fname}({ps}){r};")
        out += ["}", ""]
    return "\n".join(out)


def main() -> int:
    text = generate()
    if "--check" in sys.argv:
        ok = os.path.exists(OUT) and open(OUT).read() == text
        print("mxopt_sys.rs is up to date" if ok else "mxopt_sys.rs is out of date: run gen_rust_sys.py")
        return 0 if ok else 1
    with open(OUT, "w") as f:
        f.write(text)
    print(OUT)
    return 0


if __name__ == "__main__":
    sys.exit(main())
