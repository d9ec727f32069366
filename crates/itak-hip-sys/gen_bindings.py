#!/usr/bin/env python3
"""Writes src/lib.rs, the raw Rust binding of include/itak_hip_kv.h: one `extern "C"`
declaration per function the header declares, one `#[repr(C)]` struct per struct, one constant
per enumerator. Run from anywhere: `python crates/itak-hip-sys/gen_bindings.py`; with --check it
only reports whether src/lib.rs is what it would write (tests/test_abi_cpu.py runs that)."""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "..", "..", "include", "itak_hip_kv.h")
OUT = os.path.join(HERE, "src", "lib.rs")

SCALARS = {
    "itak_status": "itak_status", "int32_t": "i32", "uint32_t": "u32", "uint64_t": "u64",
    "uint16_t": "u16", "uint8_t": "u8", "float": "f32", "char": "c_char", "void": "c_void",
    "int": "i32",
}


def strip_comments(text):
    return re.sub(r"/\*.*?\*/", "", text, flags=re.S)


def rust_type(ctype, structs):
    """`const float *const *` -> `*const *const f32` and the like."""
    ctype = ctype.strip()
    stars = []
    # Peel pointers from the right: each '*' may be preceded by 'const' that qualifies the pointee.
    while ctype.endswith("*") or ctype.endswith("*const"):
        if ctype.endswith("*const"):
            ctype = ctype[:-len("*const")].rstrip()
        else:
            ctype = ctype[:-1].rstrip()
        stars.append(None)
    const = False
    tokens = ctype.split()
    if "const" in tokens:
        const = True
        tokens.remove("const")
    if tokens and tokens[0] == "struct":
        tokens = tokens[1:]
    base = " ".join(tokens)
    rust = SCALARS.get(base) or (base if base in structs else None)
    if rust is None:
        raise SystemExit(f"gen_bindings: unknown C type '{base}'")
    # The innermost pointer takes the pointee's constness; outer levels in this header are all
    # pointers to const pointers or plain out-pointers.
    for level in range(len(stars)):
        innermost = level == 0
        if innermost:
            rust = ("*const " if const else "*mut ") + rust
        else:
            rust = "*const " + rust if const else "*mut " + rust
    return rust


def split_decl(decl):
    """'const float *q' -> ('const float *', 'q'); arrays become fixed-size arrays."""
    decl = decl.strip()
    m = re.match(r"^(.*?)([A-Za-z_][A-Za-z0-9_]*)\s*(\[\s*(\d+)\s*\])?$", decl, flags=re.S)
    if not m:
        raise SystemExit(f"gen_bindings: cannot parse declaration '{decl}'")
    return m.group(1).strip(), m.group(2), m.group(4)


def parse(text):
    text = strip_comments(text)
    enums = []
    for body in re.findall(r"enum\s*\{(.*?)\}\s*;", text, flags=re.S):
        for name, value in re.findall(r"([A-Z][A-Z0-9_]*)\s*=\s*([0-9]+)u?", body):
            enums.append((name, int(value)))
    structs, opaque = [], []
    for name in re.findall(r"typedef\s+struct\s+(\w+)\s+\1\s*;", text):
        opaque.append(name)
    for name, body in re.findall(r"typedef\s+struct\s+(\w+)\s*\{(.*?)\}\s*\1\s*;", text, flags=re.S):
        fields = []
        for line in body.split(";"):
            line = " ".join(line.split())
            if not line:
                continue
            ctype, first, arr = split_decl(line.split(",")[0])
            names = [(first, arr)]
            for more in line.split(",")[1:]:
                names.append((more.strip(), None))
            for fname, farr in names:
                fields.append((ctype, fname, farr))
        structs.append((name, fields))
    known = set(opaque) | {n for n, _ in structs}
    functions = []
    body = re.sub(r"typedef\s+struct\s+\w+\s*\{.*?\}\s*\w+\s*;", "", text, flags=re.S)
    body = re.sub(r"enum\s*\{.*?\}\s*;", "", body, flags=re.S)
    for ret, name, args in re.findall(r"([A-Za-z_][A-Za-z0-9_ \*]*?)\b(itak_[a-z0-9_]+)\s*\(([^;{}]*?)\)\s*;",
                                      body, flags=re.S):
        ret = " ".join(ret.split())
        if ret.startswith("typedef"):
            continue
        params = []
        args = " ".join(args.split())
        if args and args != "void":
            for a in args.split(","):
                ctype, pname, _ = split_decl(a)
                params.append((ctype, pname))
        functions.append((ret, name, params))
    return enums, opaque, structs, functions, known


def render():
    enums, opaque, structs, functions, known = parse(open(HEADER).read())
    out = []
    out.append("//! Raw binding of `include/itak_hip_kv.h` (the C ABI of `libitak_hip_kv.so`), written by\n"
               "//! `gen_bindings.py` from the header: do not edit by hand. The safe wrapper over it is the\n"
               "//! `safe` module of this crate's sibling `hip-compute`; every `unsafe` of the backend lives\n"
               "//! behind these declarations (the reference's hot-path crates forbid it, `Cargo.toml:12-43`).\n"
               "#![allow(non_camel_case_types)]\n#![allow(clippy::too_many_arguments)]\n"
               "#![allow(missing_docs)]\n\n"
               "use std::os::raw::{c_char, c_void};\n\n"
               "/// Status of every call: 0 is success (`ITAK_OK`), the rest are the `ITAK_*` constants.\n"
               "pub type itak_status = i32;\n")
    for name, value in enums:
        out.append(f"pub const {name}: u32 = {value};")
    out.append("")
    for name in opaque:
        out.append(f"/// Opaque handle.\n#[repr(C)]\npub struct {name} {{\n    _private: [u8; 0],\n}}\n")
    for name, fields in structs:
        out.append("#[repr(C)]\n#[derive(Clone, Copy)]\npub struct " + name + " {")
        for ctype, fname, arr in fields:
            rt = rust_type(ctype, known)
            if arr:
                rt = f"[{rt}; {arr}]"
            out.append(f"    pub {fname}: {rt},")
        out.append("}\n")
    out.append('#[link(name = "itak_hip_kv")]\nextern "C" {')
    for ret, name, params in functions:
        args = ", ".join(f"{p}: {rust_type(t, known)}" for t, p in params)
        if ret == "void":
            out.append(f"    pub fn {name}({args});")
        else:
            out.append(f"    pub fn {name}({args}) -> {rust_type(ret, known)};")
    out.append("}")
    out.append("\npub mod safe;")
    return "\n".join(out) + "\n"


def main():
    text = render()
    if "--check" in sys.argv:
        have = open(OUT).read() if os.path.exists(OUT) else ""
        if have != text:
            print("src/lib.rs is out of date: run gen_bindings.py")
            return 1
        return 0
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    with open(OUT, "w") as f:
        f.write(text)
    print(f"wrote {OUT}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
