"""The Rust FFI crate (rust/meganeura-hip-sys, written against the headers, never compiled in
this image) against include/*.h: every symbol declared, same arity, same argument and return
types under the C -> Rust type mapping; enum constants and struct fields in step."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = ("mgn_hip.h", "mgn_bench.h", "mgn_session.h")
PRIM = {"int": "c_int", "int32_t": "i32", "uint32_t": "u32", "uint64_t": "u64", "size_t": "usize", "float": "f32",
        "char": "c_char", "uint8_t": "u8", "void": "c_void"}


def strip_comments(text):
    return re.sub(r"/\*.*?\*/", "", text, flags=re.S)


def c_type_to_rust(ty):
    """`const mgn_weight* const*` -> `*const *const mgn_weight`."""
    toks = ty.replace("*", " * ").split()
    i, const = 0, False
    if toks[0] == "const":
        const, i = True, 1
    cur = PRIM.get(toks[i], toks[i])
    i += 1
    while i < len(toks):
        assert toks[i] == "*", ty
        cur = ("*const " if const else "*mut ") + cur
        const = i + 1 < len(toks) and toks[i + 1] == "const"
        i += 2 if const else 1
    return cur


def c_prototypes():
    out = {}
    for header in HEADERS:
        text = strip_comments(open(os.path.join(ROOT, "include", header)).read())
        text = re.sub(r"typedef\s+(enum|struct)\s+\w+\s*\{.*?\}\s*\w+\s*;", "", text, flags=re.S)
        text = re.sub(r"#.*", "", text)
        for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b(mgn_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
            ret, name, args = m.group(1).strip(), m.group(2), m.group(3).strip()
            args = [] if args in ("", "void") else [re.match(r"^(.*?)\w+$", a.strip()).group(1) for a in args.split(",")]
            out[name] = ([c_type_to_rust(a) for a in args], None if ret == "void" else c_type_to_rust(ret))
    return out


def rust_prototypes():
    text = re.sub(r"//.*", "", open(os.path.join(ROOT, "rust", "meganeura-hip-sys", "src", "lib.rs")).read())
    out = {}
    for m in re.finditer(r"pub fn (mgn_\w+)\s*\(([^)]*)\)\s*(?:->\s*([^;]+?))?\s*;", text):
        name, args, ret = m.group(1), m.group(2).strip(), m.group(3)
        args = [] if not args else [a.split(":", 1)[1].strip() for a in args.split(",")]
        assert name not in out, name
        out[name] = (args, ret.strip() if ret else None)
    return text, out


def test_every_header_symbol_is_declared_with_the_same_signature():
    c, (_, r) = c_prototypes(), rust_prototypes()
    assert len(c) > 70
    assert sorted(set(c) - set(r)) == [], "missing from lib.rs"
    assert sorted(set(r) - set(c)) == [], "lib.rs declares what no header has"
    for name in sorted(c):
        assert len(c[name][0]) == len(r[name][0]), (name, "arity")
        assert c[name] == r[name], name


def test_enum_constants_and_struct_fields_match():
    rust_text, _ = rust_prototypes()
    consts = {m.group(1): int(m.group(2)) for m in re.finditer(r"pub const (MGN_\w+): \w+ = (\d+);", rust_text)}
    fields = {}
    for m in re.finditer(r"pub struct (mgn_\w+) \{(.*?)\}", rust_text, flags=re.S):
        fields[m.group(1)] = [f.split(":")[0].strip() for f in re.findall(r"pub (\w+\s*:[^,]+),", m.group(2))]
    seen_enums = 0
    for header in HEADERS:
        text = strip_comments(open(os.path.join(ROOT, "include", header)).read())
        for m in re.finditer(r"typedef\s+enum\s+\w+\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S):
            nxt = 0
            for item in [i.strip() for i in m.group(1).split(",") if i.strip()]:
                name, _, val = item.partition("=")
                nxt = int(val) if val.strip() else nxt
                assert consts.get(name.strip()) == nxt, (m.group(2), name.strip())
                nxt += 1
                seen_enums += 1
        for m in re.finditer(r"typedef\s+struct\s+\w+\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S):
            names = [re.match(r".*?(\w+)(\[\d+\])?$", f.strip()).group(1) for f in m.group(1).split(";") if f.strip()]
            assert fields.get(m.group(2)) == names, m.group(2)
    assert seen_enums > 30
    assert set(("mgn_matmul_item", "mgn_plan_info", "mgn_dispatch_info")) <= set(fields)
