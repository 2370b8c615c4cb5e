"""sage-hip-sys/src/lib.rs against include/sage_hip.h, as text (there is no Rust toolchain to build the crate with).

Both files are parsed here: every entry point of the header must be declared in the crate with the same argument
count, the same argument names in the same order and the Rust type that corresponds to the C type; every struct
with the same fields in the same order (`#[repr(C)]`); every enum value and size constant with the same number.
The header in turn equals the library's exported symbols (tests/test_host_cpu.py), so the crate binds what is built.
"""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "sage_hip.h")
CRATE = os.path.join(ROOT, "sage-hip-sys")

SCALARS = {"int": "c_int", "int32_t": "i32", "uint32_t": "u32", "int64_t": "i64", "uint64_t": "u64", "float": "f32",
           "void": "c_void", "char": "c_char"}


def c_type_to_rust(ctype, array):
    """'const sg_tensor *' -> '*const sg_tensor'; 'void **' -> '*mut *mut c_void'; 'const int32_t' + [2] as a parameter
    -> '*const i32' (an array parameter is a pointer)."""
    t = ctype.strip()
    const = t.startswith("const ")
    if const:
        t = t[len("const "):].strip()
    stars = t.count("*")
    base = t.replace("*", "").strip()
    rust = SCALARS.get(base, base)
    if array is not None:
        stars += 1
    for level in range(stars):
        rust = ("*const " if const and level == 0 else "*mut ") + rust
    return rust


def strip_c_comments(text):
    return re.sub(r"/\*.*?\*/", " ", text, flags=re.S)


def split_declarator(decl):
    """'const int32_t ker[2]' -> ('const int32_t', 'ker', '2'); 'sg_ctx **out' -> ('sg_ctx **', 'out', None)."""
    m = re.match(r"^(.*?)(\w+)\s*(?:\[(\w+)\])?$", decl.strip(), flags=re.S)
    return m.group(1).strip(), m.group(2), m.group(3)


def parse_header():
    text = strip_c_comments(open(HEADER).read())
    funcs = {}
    for m in re.finditer(r"^\s*((?:const\s+)?\w+\s*\**)\s*(sg_\w+)\s*\(([^;{]*?)\)\s*;", text, flags=re.M | re.S):
        ret, name, args = m.group(1), m.group(2), m.group(3)
        params = []
        for a in args.split(","):
            ctype, pname, arr = split_declarator(" ".join(a.split()))
            params.append((pname, c_type_to_rust(ctype, arr)))
        funcs[name] = (params, c_type_to_rust(ret, None))
    structs = {}
    for m in re.finditer(r"typedef\s+struct\s+(\w+)\s*\{(.*?)\}\s*\1\s*;", text, flags=re.S):
        fields = []
        for line in m.group(2).split(";"):
            line = " ".join(line.split())
            if not line:
                continue
            first, *more = [p.strip() for p in line.split(",")]
            ctype, fname, arr = split_declarator(first)
            names = [(fname, arr)] + [split_declarator(ctype + " " + x)[1:] for x in more]
            for fname, arr in names:
                base = c_type_to_rust(ctype, None)
                fields.append((fname, f"[{base}; {arr}]" if arr else base))
        structs[m.group(1)] = fields
    opaque = set(re.findall(r"typedef\s+struct\s+(\w+)\s+\1\s*;", text))
    enums = {}
    for m in re.finditer(r"typedef\s+enum\s+\w+\s*\{(.*?)\}", text, flags=re.S):
        value = -1
        for item in m.group(1).split(","):
            item = item.strip()
            if not item:
                continue
            if "=" in item:
                name, v = [p.strip() for p in item.split("=")]
                value = int(v, 0)
            else:
                name, value = item, value + 1
            enums[name] = value
    defines = {}
    for m in re.finditer(r"^#define\s+(SG_\w+)\s+(.+)$", text, flags=re.M):
        expr = re.sub(r"(\d)(?:ull|u)\b", r"\1", m.group(2).strip())
        defines[m.group(1)] = eval(expr, {"__builtins__": {}})
    return funcs, structs, opaque, enums, defines


def parse_crate():
    text = re.sub(r"//.*", "", open(os.path.join(CRATE, "src", "lib.rs")).read())
    funcs = {}
    block = re.search(r'extern\s+"C"\s*\{(.*)\}', text, flags=re.S).group(1)
    for m in re.finditer(r"pub\s+fn\s+(\w+)\s*\((.*?)\)\s*(?:->\s*([^;]+?))?\s*;", block, flags=re.S):
        params = []
        for a in m.group(2).split(","):
            a = " ".join(a.split())
            if a:
                pname, ptype = [p.strip() for p in a.split(":", 1)]
                params.append((pname, ptype))
        funcs[m.group(1)] = (params, (m.group(3) or "()").strip())
    structs, opaque = {}, set()
    for m in re.finditer(r"((?:#\[[^\]]*\]\s*)*)pub\s+struct\s+(\w+)\s*\{(.*?)\}", text, flags=re.S):
        attrs, name, body = m.groups()
        assert "repr(C)" in attrs, f"struct {name} is not #[repr(C)]"
        fields = []
        for f in re.split(r",(?![^\[]*\])", body):  # commas outside [T; N]
            f = " ".join(f.split())
            if f:
                fname, ftype = [p.strip() for p in f.split(":", 1)]
                fields.append((fname.replace("pub ", ""), ftype))
        if [n for n, _ in fields] == ["_private"]:
            opaque.add(name)
        else:
            structs[name] = fields
    consts = {}
    for m in re.finditer(r"pub\s+const\s+(\w+)\s*:\s*\w+\s*=\s*([^;]+);", text):
        consts[m.group(1)] = eval(m.group(2), {"__builtins__": {}})
    return funcs, structs, opaque, consts


# names the two languages cannot share: `in` is a Rust keyword
RENAMED = {"in": {"inputs", "input"}}


def test_crate_declares_every_entry_point_with_the_headers_signature():
    h_funcs, _, _, _, _ = parse_header()
    r_funcs, _, _, _ = parse_crate()
    assert len(h_funcs) >= 48
    assert sorted(h_funcs) == sorted(r_funcs), (sorted(set(h_funcs) ^ set(r_funcs)))
    assert list(h_funcs) == list(r_funcs), "the crate lists the entry points in the header's order"
    for name, (h_params, h_ret) in h_funcs.items():
        r_params, r_ret = r_funcs[name]
        assert len(h_params) == len(r_params), f"{name}: {len(h_params)} arguments in the header, {len(r_params)} in the crate"
        for (hn, ht), (rn, rt) in zip(h_params, r_params):
            assert hn == rn or rn in RENAMED.get(hn, ()), f"{name}: argument `{hn}` is `{rn}` in the crate"
            assert ht == rt, f"{name}({hn}): C type maps to `{ht}`, the crate says `{rt}`"
        assert h_ret == r_ret, f"{name}: returns `{h_ret}`, the crate says `{r_ret}`"


def test_crate_structs_have_the_headers_fields_in_order():
    _, h_structs, h_opaque, _, _ = parse_header()
    _, r_structs, r_opaque, _ = parse_crate()
    assert sorted(h_structs) == sorted(r_structs) == ["sg_adam_hyper", "sg_expr", "sg_gemm_epilogue", "sg_tensor"]
    for name, fields in h_structs.items():
        assert fields == r_structs[name], f"{name}: {fields} vs {r_structs[name]}"
    assert h_opaque == r_opaque == {"sg_ctx", "sg_graph"}


def test_crate_constants_equal_the_headers():
    _, _, _, h_enums, h_defines = parse_header()
    _, _, _, r_consts = parse_crate()
    want = dict(h_enums, **h_defines)
    assert len(want) > 80
    assert sorted(want) == sorted(r_consts), sorted(set(want) ^ set(r_consts))
    for name, value in want.items():
        assert r_consts[name] == value, f"{name}: {value} in the header, {r_consts[name]} in the crate"


def test_crate_manifest_links_the_library():
    manifest = open(os.path.join(CRATE, "Cargo.toml")).read()
    build = open(os.path.join(CRATE, "build.rs")).read()
    assert 'links = "sage_hip"' in manifest and "rustc-link-lib=dylib=sage_hip" in build
