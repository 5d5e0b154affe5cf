#!/usr/bin/env python3
"""Writes the Rust FFI declarations for include/zllm_attn.h (structs field by field, every exported function, the enums as
constants) to stdout, or into a Markdown file between the markers `<!-- ffi:begin -->` / `<!-- ffi:end -->`:

    python include/gen_rust_ffi.py                      # print
    python include/gen_rust_ffi.py --into <file.md>

The Rust side follows the conventions of the reference's own FFI layer (src/kernel/rocm/hip/ffi.rs:31-70,357-375):
`#[repr(C)]` structs, raw pointers, `c_int` status codes, the stream as an opaque pointer.
"""
from __future__ import annotations

import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "zllm_attn.h")

SCALARS = {"uint32_t": "u32", "uint64_t": "u64", "int": "c_int", "float": "f32", "uint8_t": "u8", "int8_t": "i8",
           "uint16_t": "u16", "void": "c_void", "char": "c_char", "zllm_stream_t": "*mut c_void"}


def strip_comments(text: str) -> str:
    return re.sub(r"/\*.*?\*/", "", text, flags=re.S)


def rust_type(c_type: str) -> str:
    c_type = " ".join(c_type.split())
    pointer = c_type.endswith("*")
    base = c_type.rstrip("*").strip()
    const = base.startswith("const ")
    base = base[6:] if const else base
    if base.startswith("struct "):
        base = base[7:]
    name = SCALARS.get(base) or camel(base)
    if pointer:
        return ("*const " if const else "*mut ") + name
    return name


def camel(name: str) -> str:
    return "".join(part.capitalize() for part in name.split("_"))


def parse(header_text: str):
    text = strip_comments(header_text)
    structs = []
    for body, name in re.findall(r"typedef struct \w+ \{(.*?)\}\s*(\w+);", text, flags=re.S):
        fields = []
        for decl in body.split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            c_type, names = re.match(r"(.*?[\s\*])(\w+(?:\s*,\s*\w+)*)$", decl).groups()
            for field in names.split(","):
                fields.append((field.strip(), rust_type(c_type.strip())))
        structs.append((name, fields))
    functions = []
    for ret, name, params in re.findall(r"ZLLM_API\s+([\w\s\*]+?)\s*(\w+)\(([^)]*)\);", text):
        args = []
        for param in [p.strip() for p in params.split(",")]:
            if param in ("", "void"):
                continue
            array = re.match(r"(.*?)(\w+)\[\d+\]$", param)
            if array:
                args.append((array.group(2), rust_type(array.group(1).strip() + "*")))
            else:
                c_type, arg = re.match(r"(.*?[\s\*])(\w+)$", param).groups()
                args.append((arg, rust_type(c_type.strip())))
        functions.append((name, args, None if ret.strip() == "void" else rust_type(ret.strip())))
    enums = []
    for body in re.findall(r"enum \{(.*?)\};", text, flags=re.S):
        value = 0
        for item in [i.strip() for i in body.split(",") if i.strip()]:
            if "=" in item:
                item, explicit = [x.strip() for x in item.split("=")]
                value = int(explicit, 0)
            enums.append((item, value))
            value += 1
    return structs, functions, enums


def render(structs, functions, enums) -> str:
    out = ["use std::ffi::{c_char, c_int, c_void};", ""]
    for name, value in enums:
        out.append(f"pub const {name}: c_int = {value};")
    out.append("")
    for name, fields in structs:
        out.append("#[repr(C)]")
        out.append(f"pub struct {camel(name)} {{")
        for field, ty in fields:
            field = "r#in" if field == "in" else field
            out.append(f"    pub {field}: {ty},")
        out.append("}")
        out.append("")
    out.append('extern "C" {')
    for name, args, ret in functions:
        rendered = ", ".join(f"{a}: {t}" for a, t in args)
        out.append(f"    pub fn {name}({rendered}){'' if ret is None else ' -> ' + ret};")
    out.append("}")
    return "\n".join(out) + "\n"


def main() -> None:
    block = render(*parse(open(HEADER).read()))
    if len(sys.argv) == 3 and sys.argv[1] == "--into":
        path = sys.argv[2]
        text = open(path).read()
        begin, end = "<!-- ffi:begin -->", "<!-- ffi:end -->"
        a, b = text.index(begin) + len(begin), text.index(end)
        open(path, "w").write(text[:a] + "\n```rust\n" + block + "```\n" + text[b:])
    else:
        sys.stdout.write(block)


if __name__ == "__main__":
    main()
