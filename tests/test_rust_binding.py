"""The Rust binding (rust/fusor-hip-sys/src/lib.rs) against the C header (include/fusor_hip.h).

No Rust toolchain exists in the build image, so the binding cannot be compiled here; this test is the contract
instead.  It parses both files and fails on a symbol missing on either side, a different argument count, a
different argument or return type, a different struct field name, order or type, a different enum / status /
macro value, and on a `size_of` assertion in the Rust file that disagrees with what gcc computes for the header.
"""
import os
import re
import subprocess
import tempfile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fusor_hip.h")
LIB_RS = os.path.join(ROOT, "rust", "fusor-hip-sys", "src", "lib.rs")
SAFE_RS = os.path.join(ROOT, "rust", "fusor-hip", "src", "lib.rs")
BUILD_RS = os.path.join(ROOT, "rust", "fusor-hip-sys", "build.rs")

SCALARS = {"int": "c_int", "int32_t": "i32", "uint32_t": "u32", "int64_t": "i64", "uint64_t": "u64", "size_t": "usize",
           "float": "f32", "char": "c_char", "void": "c_void"}


def _strip_c(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def _strip_rs(text):
    return re.sub(r"//[^\n]*", "", text)


def c_type_to_rust(ctype, named):
    """'const fhip_tensor4 *' -> '*const fhip_tensor4'; `named` = struct/enum/handle names of the header."""
    toks = ctype.replace("*", " * ").split()
    stars = toks.count("*")
    const = "const" in toks
    base = [t for t in toks if t not in ("*", "const")]
    assert len(base) == 1, ctype
    b = base[0]
    rust = SCALARS.get(b, b)
    assert b in SCALARS or b in named, f"unknown C type {b!r}"
    if stars == 0:
        return rust
    out = rust
    # the innermost pointer carries the const of the pointee; outer pointers are mutable
    out = ("*const " if const else "*mut ") + out
    for _ in range(stars - 1):
        out = "*mut " + out
    return out


def parse_header():
    src = _strip_c(open(HEADER).read())
    handles = re.findall(r"typedef\s+struct\s+(\w+)\s+\1\s*;", src)
    structs = {}
    for body, name in re.findall(r"typedef\s+struct\s*\{(.*?)\}\s*(\w+)\s*;", src, flags=re.S):
        fields = []
        for decl in body.split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            m = re.match(r"(.*?)(\w+)(\[(\d+)\])?$", decl)
            fields.append((m.group(2), m.group(1).strip(), int(m.group(4)) if m.group(4) else None))
        structs[name] = fields
    enums, consts = {}, {}
    for body, name in re.findall(r"(?:typedef\s+)?enum\s*\{(.*?)\}\s*(\w*)\s*;", src, flags=re.S):
        nxt = 0
        for item in body.split(","):
            item = item.strip()
            if not item:
                continue
            if "=" in item:
                key, val = [x.strip() for x in item.split("=")]
                nxt = int(val, 0)
            else:
                key = item
            consts[key] = nxt
            nxt += 1
        if name:
            enums[name] = True
    macros = {}
    for key, val in re.findall(r"#define\s+(FHIP_\w+)\s+\(?([^\n)]*)\)?", src):
        m = re.match(r"(\d+)u?\s*<<\s*(\d+)", val.strip())
        macros[key] = int(m.group(1)) << int(m.group(2)) if m else int(val.strip().rstrip("u"), 0)
    named = set(handles) | set(structs) | set(enums)
    funcs = {}
    for ret, name, args in re.findall(r"^\s*((?:const\s+)?\w+\s*\*?)\s*(\w+)\s*\(([^;{}]*?)\)\s*;", src, flags=re.M):
        params = []
        args = " ".join(args.split())
        if args != "void":
            for a in args.split(","):
                m = re.match(r"(.*?)(\w+)$", a.strip())
                params.append((m.group(2), c_type_to_rust(m.group(1).strip(), named)))
        funcs[name] = (c_type_to_rust(ret.strip(), named), params)
    return dict(handles=handles, structs=structs, enums=enums, consts=consts, macros=macros, funcs=funcs, named=named)


def parse_lib_rs():
    src = _strip_rs(open(LIB_RS).read())
    consts = {}
    for key, ty, val in re.findall(r"pub const (\w+)\s*:\s*([\w:]+)\s*=\s*([^;]+);", src):
        m = re.match(r"(\d+)\s*<<\s*(\d+)", val.strip())
        consts[key] = (ty, int(m.group(1)) << int(m.group(2)) if m else int(val.strip(), 0))
    aliases = dict(re.findall(r"pub type (\w+)\s*=\s*(\w+);", src))
    structs, repr_c = {}, set()
    for attrs, name, body in re.findall(r"((?:#\[[^\]]*\]\s*)*)pub struct (\w+)\s*\{(.*?)\n\}", src, flags=re.S):
        if "repr(C)" in attrs:
            repr_c.add(name)
        fields = []
        for decl in body.split(",\n"):
            decl = " ".join(decl.replace("pub ", "").split()).rstrip(",")
            if decl:
                fname, ftype = [x.strip() for x in decl.split(":", 1)]
                fields.append((fname, ftype))
        structs[name] = fields
    block = re.search(r'unsafe extern "C"\s*\{(.*)\n\}', src, flags=re.S).group(1)
    funcs = {}
    for name, args, ret in re.findall(r"pub fn (\w+)\s*\((.*?)\)\s*->\s*([^;]+);", block, flags=re.S):
        params = []
        for a in args.split(","):
            a = " ".join(a.split())
            if a:
                pname, ptype = [x.strip() for x in a.split(":", 1)]
                params.append((pname, ptype))
        funcs[name] = (" ".join(ret.split()), params)
    sizes = {n: int(v) for n, v in re.findall(r"size_of::<(\w+)>\(\)\s*==\s*(\d+)", src)}
    return dict(consts=consts, aliases=aliases, structs=structs, repr_c=repr_c, funcs=funcs, sizes=sizes)


def test_every_function_of_the_header_is_declared_with_the_same_signature():
    h, r = parse_header(), parse_lib_rs()
    assert len(h["funcs"]) >= 48
    assert sorted(h["funcs"]) == sorted(r["funcs"]), (
        f"missing in lib.rs: {sorted(set(h['funcs']) - set(r['funcs']))}; "
        f"not in the header: {sorted(set(r['funcs']) - set(h['funcs']))}")
    for name, (ret, params) in h["funcs"].items():
        rret, rparams = r["funcs"][name]
        assert rret == ret, f"{name}: returns {rret}, header says {ret}"
        assert len(rparams) == len(params), f"{name}: {len(rparams)} arguments, header has {len(params)}"
        for (pn, pt), (rn, rt) in zip(params, rparams):
            assert rn == pn, f"{name}: argument {rn!r} where the header has {pn!r}"
            assert rt == pt, f"{name}({pn}): {rt} where the header gives {pt}"


def test_structs_have_the_same_fields_in_the_same_order():
    h, r = parse_header(), parse_lib_rs()
    assert set(h["structs"]) <= set(r["structs"]), set(h["structs"]) - set(r["structs"])
    for name, fields in h["structs"].items():
        assert name in r["repr_c"], f"{name} is not #[repr(C)]"
        rfields = r["structs"][name]
        assert [f[0] for f in rfields] == [f[0] for f in fields], f"{name}: field order differs"
        for (fname, ctype, count), (_, rtype) in zip(fields, rfields):
            want = c_type_to_rust(ctype, h["named"])
            if count is not None:
                want = f"[{want}; {count}]"
            assert rtype == want, f"{name}.{fname}: {rtype} where the header gives {want}"
    for handle in h["handles"]:
        assert handle in r["repr_c"], f"opaque handle {handle} missing"
        assert r["structs"][handle] == [("_private", "[u8; 0]")]


def test_constants_and_enums_have_the_header_values():
    h, r = parse_header(), parse_lib_rs()
    for key, val in {**h["consts"], **h["macros"]}.items():
        assert key in r["consts"], f"{key} missing in lib.rs"
        assert r["consts"][key][1] == val, f"{key} = {r['consts'][key][1]}, header says {val}"
    for enum in h["enums"]:
        assert r["aliases"].get(enum) == "c_uint", f"enum {enum} must be an unsigned C int"
    extra = set(r["consts"]) - set(h["consts"]) - set(h["macros"])
    assert not extra, f"constants with no counterpart in the header: {extra}"


def test_struct_sizes_asserted_in_rust_are_what_gcc_computes():
    h, r = parse_header(), parse_lib_rs()
    assert set(r["sizes"]) == set(h["structs"]), "one size assertion per struct of the header"
    names = sorted(r["sizes"])
    prog = '#include <stdio.h>\n#include "fusor_hip.h"\nint main(void){\n'
    prog += "".join(f'printf("{n} %zu\\n", sizeof({n}));\n' for n in names) + "return 0;}\n"
    with tempfile.TemporaryDirectory() as tmp:
        src, exe = os.path.join(tmp, "s.c"), os.path.join(tmp, "s")
        open(src, "w").write(prog)
        subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), src, "-o", exe])
        out = subprocess.check_output([exe], text=True)
    got = {line.split()[0]: int(line.split()[1]) for line in out.splitlines()}
    assert got == r["sizes"]


def test_safe_crate_and_build_script_use_only_declared_symbols():
    r = parse_lib_rs()
    safe = _strip_rs(open(SAFE_RS).read())
    used = set(re.findall(r"\b(fhip_\w+)\s*\(", safe))
    assert used, "the safe crate calls the library"
    assert used <= set(r["funcs"]), used - set(r["funcs"])
    for must in ("fhip_flash_attention", "fhip_flash_attention_workspace_bytes", "fhip_kv_cache_append",
                 "fhip_mask_get_analytic", "fhip_malloc", "fhip_stream_create"):
        assert must in used
    # every source file of the library is compiled by build.rs
    import floneum_amd.build as fb
    build_rs = open(BUILD_RS).read()
    for src in fb.SOURCES:
        assert f'"{src}"' in build_rs, f"{src} missing from build.rs"
    assert "--offload-arch=gfx950" in build_rs and "-packed-fp32-ops" in build_rs
    assert "static=fusor_hip" in build_rs and "amdhip64" in build_rs
