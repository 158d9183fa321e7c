"""The Rust FFI crate under ffi/ against the C headers and the ctypes mirror.

No Rust toolchain exists in this image, so the crate cannot be compiled here; what can be
checked is that its `#[repr(C)]` structs and `extern "C"` declarations say exactly what
include/*.h say (names, order, types), that the struct sizes this implies equal the sizes the
C compiler and ctypes give, and that every symbol the library exports is declared."""
import ctypes as C
import os
import re
import subprocess

import pytest

from eidola_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SYS_RS = os.path.join(ROOT, "ffi", "eidola-attn-sys", "src", "lib.rs")
SAFE_RS = os.path.join(ROOT, "ffi", "eidola-attn", "src", "lib.rs")
HEADERS = [os.path.join(ROOT, "include", h) for h in ("eidola_attn.h", "eidola_sched.h")]

C_TO_RUST = {
    "uint32_t": "u32", "int32_t": "i32", "int64_t": "i64", "size_t": "usize", "float": "f32",
    "void": "()",
    "const void *": "*const c_void", "void *": "*mut c_void",
    "const int32_t *": "*const i32", "int32_t *": "*mut i32",
    "const int64_t *": "*const i64", "int64_t *": "*mut i64",
    "const float *": "*const f32", "float *": "*mut f32",
    "const char *": "*const c_char",
    "const eid_attn_desc *": "*const eid_attn_desc", "const eid_attn_args *": "*const eid_attn_args",
    "const eid_sched_config *": "*const eid_sched_config", "eid_sched **": "*mut *mut eid_sched",
    "eid_sched *": "*mut eid_sched", "const eid_sched *": "*const eid_sched",
    "eid_batch_info *": "*mut eid_batch_info",
}
RUST_SIZE = {"u32": (4, 4), "i32": (4, 4), "i64": (8, 8), "usize": (8, 8), "f32": (4, 4)}


def _strip_c_comments(text):
    return re.sub(r"/\*.*?\*/", " ", text, flags=re.S)


def _split_decl(decl):
    """'const int32_t *seq_lens' -> ('const int32_t *', 'seq_lens')"""
    decl = " ".join(decl.split())
    m = re.match(r"^(.*?)(\w+)$", decl)
    ctype, name = m.group(1).strip(), m.group(2)
    ctype = re.sub(r"\s*\*\s*", " *", ctype).replace("* *", "**").strip()
    ctype = re.sub(r" \*( \*)+", lambda mm: " " + "*" * mm.group(0).count("*"), ctype)
    return ctype, name


def c_header_model():
    structs, funcs, consts = {}, {}, {}
    for path in HEADERS:
        text = _strip_c_comments(open(path).read())
        for m in re.finditer(r"typedef struct (\w+) \{(.*?)\} (\w+);", text, flags=re.S):
            fields = [_split_decl(f) for f in m.group(2).split(";") if f.strip()]
            structs[m.group(3)] = fields
        for m in re.finditer(r"^\s*([\w ]+?[\w\*]) ?(\beid_\w+)\(([^;{]*?)\);", text, flags=re.S | re.M):
            ret = " ".join(m.group(1).split())
            ret = re.sub(r"\s*\*$", " *", ret)
            params = m.group(3).strip()
            plist = [] if params in ("", "void") else [_split_decl(p) for p in params.split(",")]
            funcs[m.group(2)] = (ret, plist)
        for m in re.finditer(r"\b(EID_\w+) = (-?\d+)", text):
            consts[m.group(1)] = int(m.group(2))
        for m in re.finditer(r"#define (EID_VERSION_\w+) (\d+)", text):
            consts[m.group(1)] = int(m.group(2))
    return structs, funcs, consts


def rust_sys_model():
    text = re.sub(r"//.*", "", open(SYS_RS).read())
    structs, funcs, consts = {}, {}, {}
    for m in re.finditer(r"#\[repr\(C\)\][^{]*?pub struct (\w+) \{(.*?)\n\}", text, flags=re.S):
        fields = []
        for f in m.group(2).split(","):
            f = f.strip()
            if not f:
                continue
            fm = re.match(r"^(?:pub )?(\w+): (.+)$", f, flags=re.S)
            fields.append((fm.group(2).strip(), fm.group(1)))
        structs[m.group(1)] = fields
    ext = re.search(r'unsafe extern "C" \{(.*)\n\}', text, flags=re.S).group(1)
    for m in re.finditer(r"pub fn (\w+)\((.*?)\)( -> ([^;]+))?;", ext, flags=re.S):
        params = [p.strip() for p in m.group(2).split(",") if p.strip()]
        plist = []
        for p in params:
            name, ty = p.split(":", 1)
            plist.append((ty.strip(), name.strip()))
        funcs[m.group(1)] = ((m.group(4) or "()").strip(), plist)
    for m in re.finditer(r"pub const (\w+): \w+ = ([^;]+);", text):
        consts[m.group(1)] = int(eval(m.group(2)))
    return structs, funcs, consts


def rust_layout(fields):
    """(size, align) of a #[repr(C)] struct whose fields are scalars or pointers."""
    off, amax = 0, 1
    for ty, _ in fields:
        size, align = (8, 8) if ty.startswith("*") else RUST_SIZE[ty]
        off = (off + align - 1) // align * align + size
        amax = max(amax, align)
    return (off + amax - 1) // amax * amax, amax


def test_structs_match_the_headers_field_for_field():
    cs, _, _ = c_header_model()
    rs, _, _ = rust_sys_model()
    for name in ("eid_attn_desc", "eid_attn_args", "eid_sched_config", "eid_batch_info"):
        want = [(C_TO_RUST[t], n) for t, n in cs[name]]
        assert rs[name] == want, name


def test_struct_sizes_match_ctypes_and_the_c_compiler(tmp_path):
    rs, _, _ = rust_sys_model()
    mirrors = {"eid_attn_desc": _lib.AttnDesc, "eid_attn_args": _lib.AttnArgs,
               "eid_sched_config": _lib.SchedConfig, "eid_batch_info": _lib.BatchInfo}
    for name, ct in mirrors.items():
        assert rust_layout(rs[name])[0] == C.sizeof(ct), name
        assert [n for _, n in rs[name]] == [f[0] for f in ct._fields_], name
    # and the C compiler's own opinion
    src = tmp_path / "sizes.c"
    src.write_text('#include <stdio.h>\n#include "eidola_attn.h"\n#include "eidola_sched.h"\n'
                   'int main(void) { printf("%zu %zu %zu %zu\\n", sizeof(eid_attn_desc), sizeof(eid_attn_args),'
                   ' sizeof(eid_sched_config), sizeof(eid_batch_info)); return 0; }\n')
    exe = tmp_path / "sizes"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    got = [int(x) for x in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()]
    assert got == [rust_layout(rs[n])[0] for n in ("eid_attn_desc", "eid_attn_args", "eid_sched_config",
                                                   "eid_batch_info")]


def test_functions_match_the_headers_argument_for_argument():
    _, cf, _ = c_header_model()
    _, rf, _ = rust_sys_model()
    assert set(cf) == set(rf)
    for name, (ret, params) in cf.items():
        want = (C_TO_RUST[ret], [(C_TO_RUST[t], n) for t, n in params])
        assert rf[name] == want, name


def test_every_exported_symbol_is_declared_and_constants_agree():
    _, rf, rc = rust_sys_model()
    _, _, cc = c_header_model()
    assert set(_lib.EXPORTS) | set(_lib.SCHED_EXPORTS) == set(rf)
    for k, v in cc.items():
        assert rc[k] == v, k
    assert rc["EID_STATIC_WORKSPACE_BYTES"] == _lib.STATIC_WORKSPACE_BYTES == 32 << 20


def test_safe_wrapper_covers_every_status_and_uses_only_declared_symbols():
    safe = open(SAFE_RS).read()
    _, rf, rc = rust_sys_model()
    for status in ("EID_ERR_INVALID_ARG", "EID_ERR_UNSUPPORTED", "EID_ERR_WORKSPACE", "EID_ERR_HIP",
                   "EID_ERR_NO_BLOCKS"):
        assert f"sys::{status} =>" in safe, status
    used = set(re.findall(r"sys::(eid_\w+)\(", safe))
    assert used <= set(rf)
    # the hot-path entry points, the scheduler and the entry point that allocates nothing
    assert {"eid_kv_write", "eid_attn_decode", "eid_attn_decode_noalloc", "eid_attn_varlen",
            "eid_lse_merge", "eid_sched_create", "eid_sched_destroy", "eid_sched_build_batch"} <= used
    assert "thiserror::Error" in safe and "impl Drop for Scheduler" in safe


@pytest.mark.parametrize("crate", ["eidola-attn-sys", "eidola-attn"])
def test_cargo_manifests_declare_a_license(crate):
    text = open(os.path.join(ROOT, "ffi", crate, "Cargo.toml")).read()
    assert re.search(r'^license = "[^"]+"', text, flags=re.M)
    assert re.search(r"^publish = false", text, flags=re.M)
    if crate == "eidola-attn-sys":
        assert 'links = "eidola_attn_hip"' in text
        build = open(os.path.join(ROOT, "ffi", crate, "build.rs")).read()
        assert "rustc-link-lib=dylib=eidola_attn_hip" in build
