"""The Rust binding kept as source (rust/hip.rs) declares exactly the functions of include/mk_hip.h, with the same
argument counts, and its repr(C) structs carry the header's fields in the header's order.  No Rust toolchain is
needed: both files are read as text."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions():
    src = open(os.path.join(ROOT, "include", "mk_hip.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    src = re.sub(r"typedef\s+struct[^;{]*\{.*?\}\s*\w+\s*;", "", src, flags=re.S)
    out = {}
    for m in re.finditer(r"\b(mk_\w+)\s*\(([^;{}]*?)\)\s*;", src, flags=re.S):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if args in ("", "void") else args.count(",") + 1
    return out


def rust_functions():
    src = open(os.path.join(ROOT, "rust", "hip.rs")).read()
    block = src[src.index('extern "C" {'):]
    block = block[:block.index("\n}\n")]
    out = {}
    for m in re.finditer(r"pub fn (mk_\w+)\(([^)]*)\)", block):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if not args else args.count(":")
    return out


def test_extern_block_matches_header():
    h, r = header_functions(), rust_functions()
    assert len(h) > 70
    assert sorted(h) == sorted(r)
    assert {k: v for k, v in h.items() if r[k] != v} == {}


def struct_fields_c(name):
    src = open(os.path.join(ROOT, "include", "mk_hip.h")).read()
    m = re.search(r"typedef\s+struct[^{;]*\{([^}]*)\}\s*" + name + r"\s*;", src, flags=re.S)
    body = re.sub(r"/\*.*?\*/", "", m.group(1), flags=re.S)
    fields = []
    for decl in body.split(";"):
        for part in decl.split(","):
            ids = re.findall(r"[A-Za-z_]\w*", re.sub(r"\[[^\]]*\]", "", part))
            if ids:
                fields.append(ids[-1])
    return fields


def struct_fields_rust(name):
    src = open(os.path.join(ROOT, "rust", "hip.rs")).read()
    m = re.search(r"pub struct " + name + r"\s*\{([^}]*)\}", src, flags=re.S)
    return re.findall(r"pub (\w+):", m.group(1))


def test_structs_match_header():
    for c, r in [("mk_expert_table", "MkExpertTable"), ("mk_bin_entry", "MkBinEntry"), ("mk_prefill_layout", "MkPrefillLayout"),
                 ("mk_prof", "MkProf")]:
        assert struct_fields_c(c) == struct_fields_rust(r), c
