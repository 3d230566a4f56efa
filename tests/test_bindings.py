"""The Rust binding crate (bindings/hf2q-hip-sys, source only: no Rust toolchain in this image) declares exactly the
entry points of include/hf2q_hip.h, with the header's parameter names in the header's order, and its #[repr(C)]
structs list the header's fields in order.  Also: the built library exports every one of them."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hf2q_hip.h")
CRATE = os.path.join(ROOT, "bindings", "hf2q-hip-sys")


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def _header_functions():
    text = _strip_comments(open(HEADER).read())
    out = {}
    for m in re.finditer(r"HQ_API\s+([^;(]+?)\b(hq_\w+)\s*\(([^)]*)\)\s*;", text, flags=re.S):
        params = [p.strip() for p in m.group(3).split(",")]
        names = [] if params == ["void"] else [re.search(r"(\w+)\s*(\[\d*\])?$", p).group(1) for p in params]
        out[m.group(2)] = names
    return out


def _rust_functions():
    text = _strip_comments(open(os.path.join(CRATE, "src", "lib.rs")).read())
    block = re.search(r'extern\s+"C"\s*\{(.*?)\n\}', text, flags=re.S).group(1)
    out = {}
    for m in re.finditer(r"pub\s+fn\s+(hq_\w+)\s*\(([^)]*)\)", block, flags=re.S):
        params = [p.strip() for p in m.group(2).split(",") if p.strip()]
        out[m.group(1)] = [p.split(":")[0].strip() for p in params]
    return out


def _header_structs():
    text = _strip_comments(open(HEADER).read())
    out = {}
    for m in re.finditer(r"typedef\s+struct\s*(\w*)\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S):
        fields = []
        for decl in m.group(2).split(";"):
            decl = decl.strip()
            if not decl:
                continue
            # "uint32_t a, b, c" / "const void* x" / "uint64_t dims[4]"
            first, *rest = [d.strip() for d in decl.split(",")]
            fields.append(re.search(r"(\w+)\s*(\[\d+\])?$", first).group(1))
            fields += [re.search(r"(\w+)", r).group(1) for r in rest]
        out[m.group(3)] = fields
    return out


def _rust_structs():
    text = _strip_comments(open(os.path.join(CRATE, "src", "lib.rs")).read())
    out = {}
    for m in re.finditer(r"#\[repr\(C\)\]\s*(?:#\[derive\([^\]]*\)\]\s*)?pub\s+struct\s+(\w+)\s*\{(.*?)\n\}", text, flags=re.S):
        out[m.group(1)] = re.findall(r"pub\s+(\w+)\s*:", m.group(2))
    return out


def test_extern_block_matches_the_header():
    h, r = _header_functions(), _rust_functions()
    assert len(h) >= 50, "the header parser lost entries"
    assert sorted(h) == sorted(r), f"only in header: {sorted(set(h) - set(r))}; only in crate: {sorted(set(r) - set(h))}"
    assert list(h) == list(r), "the crate lists the functions in the header's order"
    for name in h:
        assert h[name] == r[name], f"{name}: header {h[name]} vs crate {r[name]}"


def test_repr_c_structs_match_the_header():
    h, r = _header_structs(), _rust_structs()
    for name in ("hq_qmatmul_job", "hq_moe_ffn_layer", "hq_moe_ffn_row_scales", "hq_tq_attn_params", "hq_tqp_header", "hq_gguf_tensor_info"):
        assert name in h and name in r, name
        assert h[name] == r[name], f"{name}: header {h[name]} vs crate {r[name]}"


def test_constants_match_the_header():
    text = open(HEADER).read()
    rust = open(os.path.join(CRATE, "src", "lib.rs")).read()
    for enum_value in re.findall(r"\b(HQ_(?:Q\d_\w|F32|BF16|F16))\s*=\s*(\d+)", _strip_comments(text)):
        assert re.search(rf"\b{enum_value[0]}\s*=\s*{enum_value[1]}\b", rust), enum_value
    assert "HQ_TQ_STATIC_TMP_BYTES (4u << 20)" in text and "HQ_TQ_STATIC_TMP_BYTES: usize = 4 << 20" in rust
    assert "HQ_TQP_HEADER_BYTES 40" in text and "HQ_TQP_HEADER_BYTES: usize = 40" in rust
    assert "HQ_QMATMUL_BATCH_MAX_JOBS 4" in text and "HQ_QMATMUL_BATCH_MAX_JOBS: u32 = 4" in rust


def test_crate_files_are_present():
    for f in ("Cargo.toml", "build.rs", os.path.join("src", "lib.rs")):
        assert os.path.isfile(os.path.join(CRATE, f)), f
    assert 'links = "hf2q_hip"' in open(os.path.join(CRATE, "Cargo.toml")).read()


def test_build_rs_compiles_the_library_the_way_build_py_does():
    """build.rs runs hipcc over hf2q_amd/csrc/*.hip: its source list is the directory's, its flags are build.py's."""
    from hf2q_amd import build as hq_build

    text = open(os.path.join(CRATE, "build.rs")).read()
    sources = re.search(r"const SOURCES: &\[&str\] = &\[(.*?)\];", text, flags=re.S).group(1)
    assert re.findall(r'"([^"]+)"', sources) == hq_build.sources()
    flags = re.search(r"const FLAGS: &\[&str\] = &\[(.*?)\];", text, flags=re.S).group(1)
    assert re.findall(r'"([^"]+)"', flags) == hq_build.FLAGS
    libs = re.search(r"const LINK_LIBS: &\[&str\] = &\[(.*?)\];", text, flags=re.S).group(1)
    assert re.findall(r'"([^"]+)"', libs) == hq_build.LINK_LIBS
    strict = re.search(r"const STRICT_FP: &\[\(&str, &str\)\] = &\[(.*?)\];", text, flags=re.S).group(1)
    assert {f: [fl] for f, fl in re.findall(r'\("([^"]+)", "([^"]+)"\)', strict)} == hq_build.STRICT_FP
    assert "Command::new(&hipcc)" in text and '"-shared"' in text and "cargo:rustc-link-lib=dylib=hf2q_hip" in text


def test_extern_block_types_match_the_header():
    """Parameter and field TYPES too, not only names: every C type maps to one Rust type."""
    cmap = {"void*": "*mut c_void", "const void*": "*const c_void", "const float*": "*const f32", "float*": "*mut f32",
            "const uint32_t*": "*const u32", "uint32_t*": "*mut u32", "const uint8_t*": "*const u8", "uint8_t*": "*mut u8",
            "uint32_t": "u32", "uint64_t": "u64", "size_t": "usize", "int": "c_int", "float": "f32", "double": "f64",
            "hq_ggml_type": "hq_ggml_type", "hq_act_dtype": "hq_act_dtype", "const char*": "*const c_char",
            "size_t*": "*mut usize", "uint64_t*": "*mut u64", "double*": "*mut f64", "const char**": "*mut *const c_char",
            "const hq_tq_attn_params*": "*const hq_tq_attn_params", "const hq_tqp_header*": "*const hq_tqp_header",
            "hq_tqp_header*": "*mut hq_tqp_header", "const hq_qmatmul_job*": "*const hq_qmatmul_job",
            "const hq_moe_ffn_layer*": "*const hq_moe_ffn_layer", "const hq_moe_ffn_row_scales*": "*const hq_moe_ffn_row_scales",
            "hq_gguf**": "*mut *mut hq_gguf", "hq_gguf*": "*mut hq_gguf", "const hq_gguf*": "*const hq_gguf",
            "hq_gguf_tensor_info*": "*mut hq_gguf_tensor_info"}
    text = _strip_comments(open(HEADER).read())
    rust = _strip_comments(open(os.path.join(CRATE, "src", "lib.rs")).read())
    block = re.search(r'extern\s+"C"\s*\{(.*?)\n\}', rust, flags=re.S).group(1)
    rfn = {m.group(1): ([p.split(":", 1)[1].strip() for p in m.group(2).split(",") if p.strip()], (m.group(3) or "").strip())
           for m in re.finditer(r"pub\s+fn\s+(hq_\w+)\s*\(([^)]*)\)\s*(?:->\s*([^;]+))?;", block, flags=re.S)}
    checked = 0
    for m in re.finditer(r"HQ_API\s+([^;(]+?)\b(hq_\w+)\s*\(([^)]*)\)\s*;", text, flags=re.S):
        ret, name, params = " ".join(m.group(1).split()), m.group(2), [p.strip() for p in m.group(3).split(",")]
        ctypes_ = [] if params == ["void"] else [" ".join(re.sub(r"\b\w+\s*(\[\d*\])?$", "", p).split()).replace(" *", "*") for p in params]
        want = [cmap[c] for c in ctypes_]
        got, rret = rfn[name]
        assert got == want, f"{name}: header {ctypes_} -> {want}, crate {got}"
        want_ret = {"void": "", "int": "c_int", "size_t": "usize", "uint32_t": "u32", "uint64_t": "u64", "const char*": "*const c_char",
                    "const void*": "*const c_void"}[ret.replace(" *", "*")]
        assert rret == want_ret, f"{name}: returns {ret} vs {rret}"
        checked += 1
    assert checked >= 60
