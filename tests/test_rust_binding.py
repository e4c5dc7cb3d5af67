"""The Rust FFI crate (rust/rocmforge-mi355-sys) ships as source: no Rust toolchain exists where this library is
built.  What can be checked without one: its `extern "C"` block declares exactly the functions of include/rfq.h,
with the same number of arguments, the same argument names in the same order, compatible types, and every
enumerator of the header as a constant of the same value."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

C_TO_RUST = {
    "int": "c_int", "size_t": "usize", "float": "c_float", "void": None,
    "const void *": "*const c_void", "void *": "*mut c_void", "const float *": "*const f32", "float *": "*mut f32",
    "const uint8_t *": "*const u8", "const uint32_t *": "*const u32", "int *": "*mut c_int", "const char *": "*const c_char",
}


def c_functions():
    text = open(os.path.join(ROOT, "include", "rfq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for ret, name, args in re.findall(r"RFQ_API\s+([\w\s\*]+?)\b(rfq_\w+)\s*\(([^)]*)\)\s*;", text):
        params = []
        for a in [a.strip() for a in args.split(",")]:
            if a == "void" or not a:
                continue
            m = re.match(r"(.*?)(\w+)$", a)
            params.append((re.sub(r"\s+", " ", m.group(1)).strip().replace(" *", " *"), m.group(2)))
        out[name] = (re.sub(r"\s+", " ", ret).strip(), params)
    return out


def rust_functions():
    text = open(os.path.join(ROOT, "rust", "rocmforge-mi355-sys", "src", "lib.rs")).read()
    block = re.search(r'extern "C" \{(.*?)\n\}', text, flags=re.S).group(1)
    block = re.sub(r"//.*", "", block)
    out = {}
    for name, args, ret in re.findall(r"pub fn (rfq_\w+)\s*\(([^)]*)\)\s*(?:->\s*([^;]+))?;", block, flags=re.S):
        params = []
        for a in [a.strip() for a in args.replace("\n", " ").split(",") if a.strip()]:
            pname, ptype = [t.strip() for t in a.split(":")]
            params.append((ptype, pname))
        out[name] = ((ret or "").strip(), params)
    return out, text


def test_extern_block_matches_the_header():
    c, (r, _) = c_functions(), rust_functions()
    assert len(c) >= 30
    assert set(c) == set(r), (sorted(set(c) - set(r)), sorted(set(r) - set(c)))
    for name, (cret, cparams) in c.items():
        rret, rparams = r[name]
        assert len(cparams) == len(rparams), name
        assert C_TO_RUST[cret] == (rret or None), (name, cret, rret)
        for (ctype, cname), (rtype, rname) in zip(cparams, rparams):
            assert cname == rname, (name, cname, rname)
            assert C_TO_RUST[ctype] == rtype, (name, cname, ctype, rtype)


def test_constants_match_the_header():
    header = open(os.path.join(ROOT, "include", "rfq.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    enums = dict(re.findall(r"\b(RFQ_[A-Z0-9_]+)\s*=\s*(-?(?:0x[0-9A-Fa-f]+|\d+))", header))
    enums.update(dict(re.findall(r"#define\s+(RFQ_(?:VERSION|TABLE_F32|GEMM_ONE_PLANE))\s+(0x[0-9A-Fa-f]+|\d+)", header)))
    _, text = rust_functions()
    consts = dict(re.findall(r"pub const (RFQ_[A-Z0-9_]+): c_int = (-?(?:0x[0-9A-Fa-f]+|\d+));", text))
    assert len(enums) >= 30
    assert set(enums) == set(consts), (sorted(set(enums) - set(consts)), sorted(set(consts) - set(enums)))
    for k, v in enums.items():
        assert int(v, 0) == int(consts[k], 0), k
