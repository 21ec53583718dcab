"""The four statements of the C ABI must agree: the header (include/atenia_moe_hip.h), the Rust
`-sys` crate a maintainer of the reference adds (ffi/atenia-moe-hip-sys), the ctypes binding
(ateniaengine_amd/capi.py) and the two build recipes (csrc/Makefile, the crate's build.rs).
Rust cannot be compiled in this image, so the crate is checked as text: symbol sets, argument
counts and argument types against the header's prototypes, one stub per symbol, the source list
and the per-file contraction flags against the Makefile.  The built library must export every
symbol the header declares."""
import os
import re
import subprocess

from ateniaengine_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "atenia_moe_hip.h")
CRATE = os.path.join(ROOT, "ffi", "atenia-moe-hip-sys")
MAKEFILE = os.path.join(ROOT, "ateniaengine_amd", "csrc", "Makefile")

C_TO_RUST = {
    "int": "c_int", "float": "f32", "double": "f64", "size_t": "usize", "int64_t": "i64",
    "const char*": "*const c_char", "const float*": "*const f32", "float*": "*mut f32",
    "const void*": "*const c_void", "void*": "*mut c_void", "int32_t*": "*mut i32",
    "const int32_t*": "*const i32", "int8_t*": "*mut i8", "uint8_t*": "*mut u8", "uint16_t*": "*mut u16",
    "int64_t*": "*mut i64", "AteniaMoeLayer*": "*mut AteniaMoeLayer",
    "const AteniaMoeLayer*": "*const AteniaMoeLayer",
    "AteniaMoeLayer**": "*mut *mut AteniaMoeLayer",
    "const AteniaMoeLayerDesc*": "*const AteniaMoeLayerDesc",
}


def _norm_c(t):
    return re.sub(r"\s*\*", "*", re.sub(r"\s+", " ", t.strip()))


def header_prototypes():
    """{name: (return type, [argument types])} in Rust spelling."""
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    out = {}
    for ret, name, args in re.findall(
            r"^\s*((?:const\s+)?[A-Za-z_]\w*[\s\*]+)(\w+)\s*\(([^;{]*?)\)\s*;", text, flags=re.M):
        args = " ".join(args.split())
        types = []
        if args != "void":
            for a in args.split(","):
                m = re.match(r"(.*?)(\w+)(\[[^\]]*\])?$", a.strip())
                t = m.group(1) + ("*" if m.group(3) else "")
                types.append(C_TO_RUST[_norm_c(t)])
        out[name] = (C_TO_RUST[_norm_c(ret)], types)
    return out


def _rust_fns(text):
    out = {}
    for name, args, ret in re.findall(r"fn\s+(\w+)\s*\(([^)]*)\)\s*->\s*([^;{]+?)\s*[;{]", text):
        types = [a.split(":", 1)[1].strip() for a in args.split(",") if ":" in a]
        out[name] = (ret.strip(), types)
    return out


def rust_bindings():
    text = open(os.path.join(CRATE, "src", "lib.rs")).read()
    m = re.search(r'#\[cfg\(atenia_hip\)\]\s*#\[link\(name = "atenia_moe_hip", kind = "static"\)\]\s*'
                  r'unsafe extern "C" \{(.*?)\n\}', text, flags=re.S)
    assert m, "extern block under cfg(atenia_hip) with the static link attribute not found"
    real = _rust_fns(m.group(1))
    stubs = {}
    for body in re.findall(r"#\[cfg\(not\(atenia_hip\)\)\]\s*(?:#\[[^\]]*\]\s*)*pub unsafe (fn .*?\{)",
                           text, flags=re.S):
        stubs.update(_rust_fns(body))
    return real, stubs


def test_header_prototypes_parse():
    protos = header_prototypes()
    assert len(protos) == 38
    assert protos["atenia_moe_hip_layer_forward"] == (
        "c_int", ["*mut AteniaMoeLayer", "*const f32", "c_int", "*mut f32"])


def test_rust_extern_block_equals_the_header():
    protos = header_prototypes()
    real, stubs = rust_bindings()
    assert set(real) == set(protos), (set(real) ^ set(protos))
    for name, sig in protos.items():
        assert real[name] == sig, f"{name}: header {sig} != lib.rs {real[name]}"
    assert set(stubs) == set(protos), f"stubs missing or extra: {set(stubs) ^ set(protos)}"
    for name, sig in protos.items():
        assert stubs[name] == sig, f"stub {name}: header {sig} != lib.rs {stubs[name]}"


def test_rust_desc_struct_equals_the_header_struct():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    body = re.search(r"typedef struct AteniaMoeLayerDesc \{(.*?)\} AteniaMoeLayerDesc;", text,
                     flags=re.S).group(1)
    c_fields = []
    for decl in body.split(";"):
        decl = " ".join(decl.split())
        if decl:
            m = re.match(r"(.*?)(\w+)$", decl)
            t = _norm_c(m.group(1))
            c_fields.append((m.group(2), {"int32_t": "i32"}.get(t) or C_TO_RUST[t]))
    rust = open(os.path.join(CRATE, "src", "lib.rs")).read()
    rbody = re.search(r"#\[repr\(C\)\]\s*pub struct AteniaMoeLayerDesc \{(.*?)\n\}", rust, flags=re.S).group(1)
    r_fields = [(n, t.strip()) for n, t in re.findall(r"pub (\w+):\s*([^,]+),", rbody)]
    assert r_fields == c_fields
    assert [n for n, _ in capi.LayerDesc._fields_] == [n for n, _ in c_fields]


def test_ctypes_export_list_equals_the_header():
    protos = header_prototypes()
    assert set(capi.EXPORTS) | set(capi.REFERENCE_NAMED_EXPORTS) == set(protos)


def test_library_exports_every_declared_symbol():
    lib = capi.lib()  # raises when the library has not been built
    for name in header_prototypes():
        assert hasattr(lib, name), f"libatenia_moe_hip.so lacks {name}"
    nm = subprocess.run(["nm", "-D", "--defined-only", capi.LIB_PATH], capture_output=True,
                        text=True, check=True).stdout
    exported = {ln.split()[-1] for ln in nm.splitlines() if " T " in ln}
    assert set(header_prototypes()) <= exported


def _make_var(text, name):
    m = re.search(rf"^{name}\s*:?=\s*(.*?)(?<!\\)$", text, flags=re.M | re.S)
    return m.group(1).replace("\\\n", " ").split()


def test_build_rs_follows_the_makefile():
    mk = open(MAKEFILE).read()
    rs = open(os.path.join(CRATE, "build.rs")).read()

    def rs_list(name):
        body = re.search(rf"const {name}: &\[&str\] = &\[(.*?)\];", rs, flags=re.S).group(1)
        return re.findall(r'"([^"]+)"', body)

    assert rs_list("SOURCES") == _make_var(mk, "SRCS")
    no_contract = re.search(r"^([\w\. ]+\.o): HIPFLAGS \+= -ffp-contract=off", mk, flags=re.M).group(1)
    assert sorted(rs_list("NO_CONTRACT")) == sorted(o[:-2] + ".hip" for o in no_contract.split())
    mk_flags = [f for f in _make_var(mk, "HIPFLAGS") if f not in ("-Wall", "-Wno-unused-function")]
    mk_flags = [f.replace("$(ARCH)", "gfx950") for f in mk_flags]
    assert rs_list("HIPCC_FLAGS") == mk_flags
    assert "ar rcs" in mk and 'Command::new("ar")' in rs
    assert rs.rstrip().endswith("}") and rs.rfind("rustc-cfg=atenia_hip") > rs.rfind("rustc-link-lib")
    # every source the recipes name exists
    for s in rs_list("SOURCES"):
        assert os.path.exists(os.path.join(os.path.dirname(MAKEFILE), s))


def test_integration_doc_names_the_crate_files_not_stale_snippets():
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    for path in ("ffi/atenia-moe-hip-sys/build.rs", "ffi/atenia-moe-hip-sys/src/lib.rs",
                 "ffi/atenia-moe-hip-sys/Cargo.toml"):
        assert path in doc and os.path.exists(os.path.join(ROOT, path))
    assert "const SOURCES" not in doc, "the build recipe lives in build.rs, not in a copy in the doc"
