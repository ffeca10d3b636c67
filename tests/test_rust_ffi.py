"""The Rust FFI layer under integration/rust/ declares the C ABI of
include/mni_rocm.h faithfully: same function names, arity and argument types,
same struct fields in the same order, same constants.  (The Rust files cannot
be compiled here -- no cargo -- so this is the check that keeps them honest.)"""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = open(os.path.join(ROOT, "include", "mni_rocm.h")).read()
FFI = open(os.path.join(ROOT, "integration", "rust", "rocm_ffi.rs")).read()

C_TO_RUST = {
    "int": "c_int", "unsigned": "c_uint", "size_t": "usize", "int64_t": "i64", "int32_t": "i32", "uint32_t": "u32", "uint64_t": "u64",
    "float": "f32", "double": "f64",
    "void *": "*mut c_void", "const void *": "*const c_void", "void **": "*mut *mut c_void",
    "char *": "*mut c_char", "const char *": "*const c_char", "int *": "*mut c_int",
    "float *": "*mut f32", "int64_t": "i64", "const float *": "*const f32", "const int64_t *": "*const i64",
    "const mni_gemm_desc *": "*const MniGemmDesc", "mni_operand": "MniOperand",
}


def strip_c_comments(text):
    return re.sub(r"//[^\n]*", "", re.sub(r"/\*.*?\*/", "", text, flags=re.S))


def c_type(decl):
    """'const float *bias' -> 'const float *' ; 'int64_t M' -> 'int64_t'"""
    decl = decl.strip()
    m = re.match(r"^(.*?)(\w+)$", decl)
    base = m.group(1).strip() if m and m.group(1).strip() else decl
    base = re.sub(r"\s*\*\s*", " *", base).replace("* *", "**").strip()
    return re.sub(r"\s+", " ", base)


def header_functions():
    text = strip_c_comments(HEADER)
    out = {}
    for ret, star, name, args in re.findall(r"\n\s*((?:const )?\w+)\s*(\*?)\s*(mni_rocm_\w+)\s*\(([^)]*)\)\s*;", text):
        args = args.strip()
        params = [] if args in ("", "void") else [c_type(a) for a in args.split(",")]
        out[name] = ((ret + " *") if star else ret, params)
    return out


def rust_functions():
    block = re.search(r'extern "C" \{(.*?)\n\}', FFI, flags=re.S).group(1)
    out = {}
    for name, args, ret in re.findall(r"pub fn (\w+)\((.*?)\)\s*(?:->\s*([^;]+))?;", block, flags=re.S):
        params = [a.split(":", 1)[1].strip() for a in args.split(",") if a.strip()]
        out[name] = ((ret or "()").strip(), params)
    return out


def header_struct(name):
    body = [b for b, n in re.findall(r"typedef struct \{(.*?)\}\s*(\w+);", strip_c_comments(HEADER), flags=re.S) if n == name][0]
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        ctype = c_type(decl.split(",")[0])
        for piece in decl.split(","):
            fields.append((re.search(r"(\w+)\s*$", piece).group(1), ctype))
    return fields


def rust_struct(name):
    body = re.search(r"pub struct %s \{(.*?)\}" % name, FFI, flags=re.S).group(1)
    return [(n, t.strip()) for n, t in re.findall(r"pub (\w+):\s*([^,\n]+),", body)]


def test_every_rust_declaration_matches_the_header():
    c_fns, r_fns = header_functions(), rust_functions()
    assert len(r_fns) >= 20
    for name, (r_ret, r_params) in r_fns.items():
        assert name in c_fns, "%s is declared in rocm_ffi.rs but not in mni_rocm.h" % name
        c_ret, c_params = c_fns[name]
        assert [C_TO_RUST[p] for p in c_params] == r_params, "%s: %s vs %s" % (name, c_params, r_params)
        assert C_TO_RUST[c_ret] == r_ret, "%s returns %s vs %s" % (name, c_ret, r_ret)


def test_the_calls_the_arms_make_are_all_declared():
    used = set()
    for dirpath, _, files in os.walk(os.path.join(ROOT, "integration", "rust")):
        for f in files:
            if f.endswith(".rs") and f != "rocm_ffi.rs":
                used |= set(re.findall(r"\b(mni_rocm_\w+)\s*\(", open(os.path.join(dirpath, f)).read()))
    assert used and used <= set(rust_functions()), sorted(used - set(rust_functions()))


def test_broadcast_gradients_are_reduced_by_the_general_device_sum():
    # matmul_backward and add_backward sum a gradient over every broadcast dim, interior ones of extent 1 included
    # (utils.rs:39-66): the arms hand both shapes to mni_rocm_unbroadcast and never guess a (rows, cols) column sum
    for rel in ("ops/matmul_rocm.rs", "ops/elementwise_rocm.rs"):
        text = open(os.path.join(ROOT, "integration", "rust", rel)).read()
        back = text[text.index("_backward("):]
        assert "mni_rocm_unbroadcast(" in text and "mni_rocm_colsum(" not in back, rel
        assert "to_host(" not in back, rel  # (no host round trip for a broadcast gradient)


def test_structs_have_the_headers_fields_in_order():
    for c_name, r_name in (("mni_operand", "MniOperand"), ("mni_gemm_desc", "MniGemmDesc")):
        c_fields, r_fields = header_struct(c_name), rust_struct(r_name)
        assert [n.lower() for n, _ in c_fields] == [n for n, _ in r_fields]
        assert [C_TO_RUST[t] for _, t in c_fields] == [t for _, t in r_fields], (c_fields, r_fields)
    assert "#[repr(C)]" in FFI.split("pub struct MniOperand")[0][-80:]
    assert "#[repr(C)]" in FFI.split("pub struct MniGemmDesc")[0][-80:]


def test_constants_have_the_headers_values():
    c_defs = dict(re.findall(r"#define (MNI_\w+) (\d+)", HEADER))
    for enum in re.findall(r"enum \{(.*?)\}", strip_c_comments(HEADER), flags=re.S):
        c_defs.update(re.findall(r"(MNI_\w+) = (\d+)", enum))
    r_consts = dict(re.findall(r"pub const (MNI_\w+): \w+ = (\d+);", FFI))
    assert len(r_consts) >= 9
    for name, value in r_consts.items():
        assert c_defs.get(name) == value, name


def test_patches_name_files_that_exist_in_this_directory():
    patch = open(os.path.join(ROOT, "integration", "rust", "rocm_feature.patch")).read()
    for path in re.findall(r'#\[path = "(\w+\.rs)"\]', patch):
        found = any(path in files for _, _, files in os.walk(os.path.join(ROOT, "integration", "rust")))
        assert found, path
    loader = open(os.path.join(ROOT, "integration", "native-loader.rocm.patch")).read()
    assert "libamdhip64.so" in loader and "linux-x64-gnu-rocm" in loader
