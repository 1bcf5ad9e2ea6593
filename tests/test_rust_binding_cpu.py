"""The Rust crate under rust/candle-hip-moe cannot be compiled in this image (no cargo / rustc), so its FFI
declarations are held to the C header mechanically: the `#[repr(C)] struct MoeDesc` must list the fields of `moe_desc`
in the same order with matching types, and every function of its `extern "C"` block must exist in
include/candle_amd_moe.h with the same return type and the same parameter types in the same order."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "candle_amd_moe.h")
LIB_RS = os.path.join(ROOT, "rust", "candle-hip-moe", "src", "lib.rs")
CARGO = os.path.join(ROOT, "rust", "candle-hip-moe", "Cargo.toml")
BUILD_RS = os.path.join(ROOT, "rust", "candle-hip-moe", "build.rs")

# canonical spelling of a type: (pointer depth with constness of the pointee chain, base)
C_BASE = {"int64_t": "i64", "int32_t": "i32", "int": "i32", "uint64_t": "u64", "float": "f32", "double": "f64", "char": "c_char",
          "void": "c_void", "moe_layer": "MoeLayer", "moe_qlinear": "MoeQLinear", "moe_gguf": "MoeGguf", "moe_desc": "MoeDesc"}


def strip_c_comments(text):
    return re.sub(r"/\*.*?\*/", " ", text, flags=re.S)


def canon_c(t):
    """'const void* const*' -> '*const *const c_void'; 'moe_layer**' -> '*mut *mut MoeLayer'; 'int64_t' -> 'i64'."""
    toks = re.findall(r"\*|\w+", t)
    base, i, const_base = None, 0, False
    while toks[i] == "const" or base is None:
        if toks[i] == "const":
            const_base = True
        else:
            base = toks[i]
        i += 1
        if i >= len(toks):
            break
    ptrs = []   # constness of what each '*' points to, innermost first
    pointee_const = const_base
    while i < len(toks):
        if toks[i] == "*":
            ptrs.append(pointee_const)
            pointee_const = False
        elif toks[i] == "const":
            pointee_const = True
        i += 1
    out = C_BASE[base]
    for c in ptrs:
        out = ("*const " if c else "*mut ") + out
    return out


def canon_rust(t):
    return re.sub(r"\s+", " ", t.strip())


def split_params(s):
    s = s.strip()
    if s in ("", "void"):
        return []
    return [p.strip() for p in s.split(",")]


def c_functions():
    text = strip_c_comments(open(HEADER).read())
    text = re.sub(r"#.*", "", text)
    fns = {}
    for m in re.finditer(r"([\w\s\*]+?)\b(moe_\w+)\s*\(([^)]*)\)\s*;", text):
        ret, name, params = m.group(1).strip(), m.group(2), m.group(3)
        ptypes = []
        for p in split_params(params):
            p = re.sub(r"\[\d*\]", "*", p)                       # array parameter = pointer
            ptype = re.sub(r"\b\w+\s*$", "", p) if not p.rstrip().endswith("*") else p   # drop the parameter's name
            ptypes.append(canon_c(ptype))
        fns[name] = (canon_c(ret) if ret != "void" else "()", ptypes)
    return fns


def c_desc_fields():
    text = strip_c_comments(open(HEADER).read())
    body = re.search(r"typedef struct \{(.*?)\}\s*moe_desc\s*;", text, flags=re.S).group(1)
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        m = re.match(r"(.*?)(\w+)$", decl, flags=re.S)
        fields.append((m.group(2), canon_c(m.group(1))))
    return fields


def rust_items():
    text = re.sub(r"//.*", "", open(LIB_RS).read())
    body = re.search(r"#\[repr\(C\)\]\s*pub struct MoeDesc \{(.*?)\}", text, flags=re.S).group(1)
    fields = [(m.group(1), canon_rust(m.group(2))) for m in re.finditer(r"pub (\w+)\s*:\s*([^,]+),", body)]
    ext = re.search(r'extern "C" \{(.*?)\n    \}', text, flags=re.S).group(1)
    fns = {}
    for m in re.finditer(r"pub fn (\w+)\s*\(([^)]*)\)\s*(?:->\s*([^;]+))?;", ext):
        params = [canon_rust(p.split(":", 1)[1]) for p in split_params(m.group(2))]
        fns[m.group(1)] = (canon_rust(m.group(3)) if m.group(3) else "()", params)
    return fields, fns


def test_moe_desc_layout_matches_the_header():
    c_fields = c_desc_fields()
    r_fields, _ = rust_items()
    assert len(c_fields) == 21
    assert r_fields == c_fields


def test_extern_block_matches_the_header():
    c_fns = c_functions()
    _, r_fns = rust_items()
    assert len(r_fns) >= 20
    for name, sig in r_fns.items():
        assert name in c_fns, "%s is declared in lib.rs but not in the header" % name
        assert sig == c_fns[name], (name, sig, c_fns[name])
    # the entry points a drop-in needs are all bound
    for name in ("moe_layer_create", "moe_layer_forward", "moe_layer_destroy", "moe_layer_create_from_gguf", "moe_qlinear_create",
                 "moe_qlinear_forward", "moe_qlinear_create_from_gguf", "moe_rms_norm", "moe_last_error"):
        assert name in r_fns


def test_opaque_handles_and_trait_impls_are_present():
    text = open(LIB_RS).read()
    for item in ("impl CustomOp1 for HipSparseMoe", "impl Module for HipSparseMoe", "impl Drop for HipSparseMoe",
                 "impl CustomOp1 for HipQMatMul", "impl Module for HipQMatMul", "impl Drop for HipQMatMul",
                 "impl CustomOp1 for HipRmsNorm", "unsafe impl Send for HipSparseMoe", "unsafe impl Sync for HipSparseMoe"):
        assert item in text, item
    assert '"qmatmul"' in text          # the op name of candle-core/src/quantized/mod.rs:470-473
    # QTensor::data() returns Result<Cow<[u8]>>: the Cow has to be bound to a name that outlives the FFI call
    assert re.search(r"let data = w\.data\(\)\?;", text) and "bytes.push(w1.data()?)" in text
    cargo = open(CARGO).read()
    assert 'package = "candle-core"' in cargo and 'links = "candle_amd_moe"' in cargo
    assert "rustc-link-lib=dylib=candle_amd_moe" in open(BUILD_RS).read()
