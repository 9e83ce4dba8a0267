"""The Rust side of the boundary (rust/rbmoe) cannot be compiled where this library is built (no Rust toolchain),
so its raw declarations are at least held against `include/rbmoe.h` as text: the same functions with the same number
and kinds of arguments, the same constants, the same struct fields in the same order.  No GPU."""
import os
import re

from conftest import ROOT

HEADER = open(os.path.join(ROOT, "include", "rbmoe.h")).read()
SYS = open(os.path.join(ROOT, "rust", "rbmoe", "src", "sys.rs")).read()


def strip_comments(text, rust=False):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//.*", " ", text)


def c_kind(decl):
    """'ptr' for pointers, else the scalar's width class."""
    decl = decl.strip()
    if "*" in decl:
        return "ptr"
    base = decl.rsplit(" ", 1)[0] if " " in decl else decl
    return {"int32_t": "i32", "int": "i32", "size_t": "usize", "float": "f32", "double": "f64", "uint64_t": "u64"}[base.replace("const ", "").strip()]


def rust_kind(ty):
    ty = ty.strip()
    if ty.startswith("*"):
        return "ptr"
    return {"i32": "i32", "c_int": "i32", "usize": "usize", "f32": "f32", "f64": "f64", "u64": "u64"}[ty]


def c_functions():
    text = strip_comments(HEADER)
    out = {}
    for m in re.finditer(r"\b(int|void|const char\*)\s+(rbmoe_\w+)\s*\(([^)]*)\)\s*;", text):
        args = [a for a in (s.strip() for s in m.group(3).split(",")) if a and a != "void"]
        out[m.group(2)] = (m.group(1), [c_kind(a) for a in args])
    return out


def rust_functions():
    text = strip_comments(SYS, rust=True)
    out = {}
    for m in re.finditer(r"pub fn (rbmoe_\w+)\s*\(([^)]*)\)\s*(->\s*([^;]+))?;", text):
        args = [a for a in (s.strip() for s in m.group(2).split(",")) if a]
        ret = (m.group(4) or "").strip()
        out[m.group(1)] = ({"c_int": "int", "": "void", "*const c_char": "const char*"}[ret],
                           [rust_kind(a.split(":", 1)[1]) for a in args])
    return out


def test_every_entry_point_is_declared_with_the_same_shape():
    c, r = c_functions(), rust_functions()
    assert len(c) >= 35
    assert sorted(c) == sorted(r)
    for name in c:
        assert c[name] == r[name], (name, c[name], r[name])


def test_constants_agree():
    consts = dict((m.group(1), int(m.group(2))) for m in
                  re.finditer(r"pub const (RBMOE_\w+):\s*\w+\s*=\s*(\d+);", SYS))
    header = strip_comments(HEADER)
    c_consts = dict((m.group(1), int(m.group(2))) for m in re.finditer(r"\b(RBMOE_[A-Z0-9_]+)\s*=\s*(\d+)", header))
    c_consts.update((m.group(1), int(m.group(2))) for m in re.finditer(r"#define\s+(RBMOE_[A-Z0-9_]+)\s+(\d+)", header))
    shared = set(consts) & set(c_consts)
    assert {"RBMOE_OK", "RBMOE_NULL_POINTER", "RBMOE_I8", "RBMOE_W_NORM", "RBMOE_NUM_STAGES"} <= shared
    for name in shared:
        assert consts[name] == c_consts[name], name
    # every status, dtype and weight id of the header exists on the Rust side
    wanted = [n for n in c_consts if not n.startswith("RBMOE_STAGE_") and n != "RBMOE_H"]
    assert not [n for n in wanted if n not in consts]


def struct_fields_c(name):
    body = re.search(r"typedef struct %s\s*\{(.*?)\}\s*%s\s*;" % (name, name), strip_comments(HEADER), flags=re.S).group(1)
    return [re.sub(r"[\s\*]+", " ", f).strip().split(" ")[-1] for f in body.split(";") if f.strip()]


def struct_fields_rust(name):
    body = re.search(r"pub struct %s\s*\{(.*?)\}" % name, strip_comments(SYS), flags=re.S).group(1)
    return [f.strip().split(":")[0].replace("pub ", "").strip() for f in body.split(",") if f.strip()]


def test_struct_layouts_agree():
    for name in ("rbmoe_config", "rbmoe_routing"):
        assert struct_fields_c(name) == struct_fields_rust(name), name
