"""The Rust binding shown in the integration guide against include/zllm_attn.h: every structure field by field (name, order, type), every
exported function (name, argument types, return type) and every enum constant.  A binding written from a stale doc
passes structures of the wrong size, so any difference fails here.  Both sides are parsed in this file, independently
of the generator that writes the doc's block (include/gen_rust_ffi.py)."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

C_TO_RUST = {"uint32_t": "u32", "uint64_t": "u64", "int": "c_int", "float": "f32", "uint8_t": "u8", "int8_t": "i8", "uint16_t": "u16",
             "void": "c_void", "char": "c_char"}


def _rust_of(c_type):
    c_type = " ".join(c_type.split())
    if c_type == "zllm_stream_t":
        return "*mut c_void"
    stars = c_type.count("*")
    base = c_type.replace("*", "").strip()
    const = base.startswith("const ")
    base = base[len("const "):] if const else base
    if base.startswith("zllm_"):
        base = "".join(w.capitalize() for w in base.split("_"))
    else:
        base = C_TO_RUST[base]
    assert stars <= 1
    return (("*const " if const else "*mut ") if stars else "") + base


def _header():
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "zllm_attn.h")).read(), flags=re.S)
    structs = {}
    for body, name in re.findall(r"typedef struct \w+ \{(.*?)\}\s*(\w+);", text, flags=re.S):
        fields = []
        for decl in filter(None, (" ".join(d.split()) for d in body.split(";"))):
            names = re.search(r"(\w+(\s*,\s*\w+)*)$", decl).group(1)
            c_type = decl[: len(decl) - len(names)].strip()
            fields += [(n.strip(), _rust_of(c_type)) for n in names.split(",")]
        structs["".join(w.capitalize() for w in name.split("_"))] = fields
    functions = {}
    for ret, name, params in re.findall(r"ZLLM_API\s+([\w\s\*]+?)\s*(\w+)\(([^)]*)\);", text):
        args = []
        for param in filter(lambda p: p not in ("", "void"), (p.strip() for p in params.split(","))):
            param = re.sub(r"(\w+)\[\d+\]$", r"* \1", param)  # array parameter = pointer
            arg = re.search(r"(\w+)$", param).group(1)
            args.append(_rust_of(param[: len(param) - len(arg)].strip()))
        functions[name] = (args, None if ret.strip() == "void" else _rust_of(ret.strip()))
    constants = {}
    for body in re.findall(r"enum \{(.*?)\};", text, flags=re.S):
        value = 0
        for item in filter(None, (i.strip() for i in body.split(","))):
            if "=" in item:
                item, explicit = (x.strip() for x in item.split("="))
                value = int(explicit, 0)
            constants[item] = value
            value += 1
    return structs, functions, constants


def _doc():
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    block = text[text.index("<!-- ffi:begin -->"): text.index("<!-- ffi:end -->")]
    structs = {}
    for name, body in re.findall(r"#\[repr\(C\)\]\s*pub struct (\w+) \{(.*?)\n\}", block, flags=re.S):
        structs[name] = [(f.replace("r#", ""), t.strip()) for f, t in re.findall(r"pub ([\w#]+): ([^,\n]+),", body)]
    functions = {}
    extern = re.search(r'extern "C" \{(.*?)\n\}', block, flags=re.S).group(1)
    for name, params, ret in re.findall(r"pub fn (\w+)\(([^)]*)\)(?: -> ([^;]+))?;", extern):
        args = [p.split(":", 1)[1].strip() for p in params.split(",") if p.strip()]
        functions[name] = (args, ret.strip() if ret else None)
    constants = {name: int(value) for name, value in re.findall(r"pub const (\w+): c_int = (\d+);", block)}
    return structs, functions, constants


def test_rust_structs_match_the_header_field_by_field():
    header, doc = _header()[0], _doc()[0]
    assert sorted(header) == sorted(doc)
    for name, fields in header.items():
        assert doc[name] == fields, name


def test_rust_extern_block_declares_every_exported_function():
    header, doc = _header()[1], _doc()[1]
    assert sorted(header) == sorted(doc)
    for name, signature in header.items():
        assert doc[name] == signature, name


def test_rust_constants_match_the_enums():
    assert _header()[2] == _doc()[2]


def test_the_parsers_see_the_whole_surface():
    """Guards the test itself: the known structures and entry points are found, with the fields a stale doc once lacked."""
    structs, functions, constants = _header()
    assert {"ZllmGqaDecodeArgs", "ZllmGqaPrefillArgs", "ZllmMlaDecodeArgs", "ZllmGqaPrologueArgs", "ZllmScatterArgs", "ZllmMlaLayerRecord"} <= set(structs)
    assert [f for f, _ in structs["ZllmGqaDecodeArgs"]][-3:] == ["gate", "gate_cols", "gate_dtype"]
    assert ("in", "*const c_void") in structs["ZllmScatterArgs"]
    assert {"zllm_attn_gqa_prologue", "zllm_attn_scatter_rows", "zllm_kv_mla_layer_read", "zllm_attn_key_range", "zllm_kv_ring_write_plan"} <= set(functions)
    assert functions["zllm_attn_gqa_decode"] == (["*const ZllmGqaDecodeArgs", "*mut c_void"], "c_int")
    assert constants["ZLLM_MLA_PROJECT"] == 8
    from zllm_amd import capi

    assert set(functions) == set(capi.SYMBOLS)
