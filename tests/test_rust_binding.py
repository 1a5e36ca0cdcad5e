"""The Rust FFI crate (rust/izwi-qmm-sys) against the C headers, as text: no Rust toolchain is needed.

Every prototype of include/*.h must be declared in the crate's `extern "C"` block and nothing else,
with the same number of arguments and, argument by argument and for the result, the same base type,
pointer depth and constness at every level; the `#[repr(C)]` structs must list the headers' fields in
order with matching types; the constants must carry the headers' values; and the safe crate
(rust/izwi-qmm) may only name functions the -sys crate declares."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = ["include/izwi_qmm.h", "include/izwi_gguf.h", "include/izwi_decode_ops.h"]
SYS = "rust/izwi-qmm-sys/src/lib.rs"
SAFE = "rust/izwi-qmm/src/lib.rs"

C_TO_RUST = {"int": "c_int", "int32_t": "i32", "int64_t": "i64", "uint64_t": "u64", "uint32_t": "u32", "uint16_t": "u16",
             "uint8_t": "u8", "float": "f32", "double": "f64", "void": "c_void", "char": "c_char", "size_t": "usize",
             "izwi_qmm_weight": "IzwiQmmWeight", "izwi_qmm_weight_info": "IzwiQmmWeightInfo",
             "izwi_qmm_profile_snapshot": "IzwiQmmProfileSnapshot", "izwi_qmm_chain": "IzwiQmmChain",
             "izwi_qmm_chain_step": "IzwiQmmChainStep", "izwi_gguf": "IzwiGguf",
             "izwi_gguf_tensor_info": "IzwiGgufTensorInfo"}


def read(rel):
    with open(os.path.join(ROOT, rel)) as f:
        return f.read()


def strip_c_comments(s):
    return re.sub(r"/\*.*?\*/", "", s, flags=re.S)


def c_type(text):
    """'const float* const*' -> ('f32', [True, True]): the Rust name of the base type and, from the
    innermost pointer outwards, whether what each pointer points to is const."""
    toks = re.findall(r"\*|const|[A-Za-z_]\w*", text)
    i, base_const = 0, False
    if toks[i] == "const":
        base_const, i = True, i + 1
    base = toks[i]
    i += 1
    if i < len(toks) and toks[i] == "const":
        base_const, i = True, i + 1
    ptr_const = []
    while i < len(toks):
        assert toks[i] == "*", text
        i += 1
        c = False
        if i < len(toks) and toks[i] == "const":
            c, i = True, i + 1
        ptr_const.append(c)
    pointee_const = ([base_const] + ptr_const[:-1]) if ptr_const else []
    return C_TO_RUST[base], pointee_const


def rust_type(text):
    """'*const *mut f32' -> ('f32', [False, True]) in the same convention as c_type."""
    toks = text.split()
    consts = []
    while toks and toks[0] in ("*const", "*mut"):
        consts.append(toks.pop(0) == "*const")
    assert len(toks) == 1, text
    return toks[0], list(reversed(consts))


def c_prototypes():
    out = {}
    for h in HEADERS:
        s = strip_c_comments(read(h))
        for m in re.finditer(r"^([A-Za-z_][\w\s\*]*?)\b(izwi_\w+)\s*\(([^;{]*?)\)\s*;", s, flags=re.M):
            ret, name, args = m.group(1).strip(), m.group(2), " ".join(m.group(3).split())
            parsed = []
            if args and args != "void":
                for a in args.split(","):
                    mm = re.match(r"^(.*?)([A-Za-z_]\w*)$", a.strip())
                    parsed.append(c_type(mm.group(1)))
            assert name not in out, f"{name} is declared twice"
            out[name] = (None if ret == "void" else c_type(ret), parsed)
    return out


def rust_prototypes():
    s = re.sub(r"//.*", "", read(SYS))
    block = re.search(r'extern "C" \{(.*)\n\}', s, flags=re.S).group(1)
    out = {}
    for m in re.finditer(r"pub fn (\w+)\s*\((.*?)\)\s*(?:->\s*([^;]+?))?\s*;", block, flags=re.S):
        name, args, ret = m.group(1), " ".join(m.group(2).split()), m.group(3)
        parsed = []
        if args:
            for a in args.split(","):
                a = a.strip()
                if a:
                    parsed.append(rust_type(a.split(":", 1)[1].strip()))
        assert name not in out, f"{name} is declared twice in the extern block"
        out[name] = (None if ret is None else rust_type(ret.strip()), parsed)
    return out


def test_extern_block_declares_exactly_the_headers_functions():
    c, r = c_prototypes(), rust_prototypes()
    assert len(c) >= 80  # the three headers were found and parsed
    missing = sorted(set(c) - set(r))
    extra = sorted(set(r) - set(c))
    assert not missing, f"not declared in {SYS}: {missing}"
    assert not extra, f"declared in {SYS} but in no header: {extra}"


def test_every_argument_and_result_matches():
    c, r = c_prototypes(), rust_prototypes()
    problems = []
    for name in sorted(set(c) & set(r)):
        (cret, cargs), (rret, rargs) = c[name], r[name]
        if cret != rret:
            problems.append(f"{name}: result {cret} in the header, {rret} in Rust")
        if len(cargs) != len(rargs):
            problems.append(f"{name}: {len(cargs)} arguments in the header, {len(rargs)} in Rust")
            continue
        for i, (ca, ra) in enumerate(zip(cargs, rargs)):
            if ca != ra:
                problems.append(f"{name}: argument {i} is {ca} in the header, {ra} in Rust")
    assert not problems, "\n".join(problems)


def c_structs():
    out = {}
    for h in HEADERS:
        s = strip_c_comments(read(h))
        for m in re.finditer(r"typedef struct (\w+) \{(.*?)\} (\w+);", s, flags=re.S):
            fields = []
            for decl in m.group(2).split(";"):
                decl = " ".join(decl.split())
                if not decl:
                    continue
                mm = re.match(r"^(.*?)([A-Za-z_]\w*)(\[(\w+)\])?$", decl)
                base, consts = c_type(mm.group(1))
                fields.append((mm.group(2), base, consts, mm.group(4)))
            out[m.group(3)] = fields
    return out


def rust_structs():
    s = re.sub(r"//.*", "", read(SYS))
    out = {}
    for m in re.finditer(r"#\[repr\(C\)\]\s*(?:#\[derive\([^\]]*\)\]\s*)?pub struct (\w+) \{(.*?)\n\}", s, flags=re.S):
        fields = []
        for decl in m.group(2).split(",\n"):
            decl = " ".join(decl.split()).rstrip(",")
            if not decl or decl.startswith("_private"):
                continue
            name, ty = decl.replace("pub ", "", 1).split(":", 1)
            ty = ty.strip()
            arr = None
            am = re.match(r"^\[(.*); (\w+)\]$", ty)
            if am:
                ty, arr = am.group(1).strip(), am.group(2)
            base, consts = rust_type(ty)
            fields.append((name.strip(), base, consts, arr))
        out[m.group(1)] = fields
    return out


def test_repr_c_structs_match_the_headers():
    c, r = c_structs(), rust_structs()
    for cname, fields in c.items():
        rname = C_TO_RUST[cname]
        assert rname in r, f"struct {rname} (for {cname}) is missing"
        assert fields == r[rname], f"{cname}: header {fields} != Rust {r[rname]}"


def test_constants_carry_the_headers_values():
    text = "\n".join(strip_c_comments(read(h)) for h in HEADERS)
    values = {k: int(v) for k, v in re.findall(r"\b(IZWI_\w+)\s*=\s*(-?\d+)", text)}
    values.update({k: int(v) for k, v in re.findall(r"#define\s+(IZWI_\w+)\s+(-?\d+)\b", text)})
    rust = {k: int(v) for k, v in re.findall(r"pub const (IZWI_\w+): \w+ = (-?\d+);", read(SYS))}
    assert len(rust) >= 20
    for k, v in rust.items():
        assert k in values, f"{k} is not a constant of the headers"
        assert values[k] == v, f"{k}: {values[k]} in the header, {v} in Rust"


def test_safe_crate_names_only_declared_functions():
    declared = set(rust_prototypes())
    used = set(re.findall(r"\bsys::(izwi_\w+)\b", read(SAFE)))
    assert len(used) >= 20
    assert not (used - declared), sorted(used - declared)
