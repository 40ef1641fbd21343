"""The Rust binding text (local-hip/src/ffi.rs) against the C header (include/local_hip.h), without a Rust toolchain:
every LH_API function has exactly one `pub fn` with the same name, the same number of arguments in the same order
with the same names, and argument / return types that correspond; the enum values and constants agree; the built
library exports every function ffi.rs declares; and ffi.rs is what local-hip/gen_ffi.py generates from the header
as it stands.  The header side is parsed here independently of the generator (a bug in its parser must not be able to
hide itself)."""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "local_hip.h")
FFI = os.path.join(ROOT, "local-hip", "src", "ffi.rs")

# C spelling (whitespace squeezed, '*' attached to the type) -> Rust spelling
TYPE_MAP = {
    "int": "c_int", "float": "f32", "size_t": "usize", "uint32_t": "u32", "uint64_t": "u64",
    "lh_dtype": "lh_dtype", "lh_quant": "lh_quant",
    "void*": "*mut c_void", "const void*": "*const c_void", "char*": "*mut c_char", "const char*": "*const c_char",
    "float*": "*mut f32", "const float*": "*const f32", "uint32_t*": "*mut u32", "const uint32_t*": "*const u32",
    "uint8_t*": "*mut u8", "const uint8_t*": "*const u8", "uint16_t*": "*mut u16", "const uint16_t*": "*const u16",
}
for _h in ("lh_context", "lh_buffer", "lh_batch", "lh_event", "lh_graph"):
    TYPE_MAP[f"{_h}*"] = f"*mut {_h}"
    TYPE_MAP[f"const {_h}*"] = f"*const {_h}"
    TYPE_MAP[f"{_h}**"] = f"*mut *mut {_h}"
    TYPE_MAP[f"const {_h}* const*"] = f"*const *const {_h}"
    TYPE_MAP[f"{_h}* const*"] = f"*const *mut {_h}"


def c_functions():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    fns = []
    for m in re.finditer(r"LH_API\s+([\w\s\*]+?)\b(lh_\w+)\s*\(([^)]*)\)\s*;", text):
        ret = " ".join(m.group(1).replace("*", " * ").split()).replace(" *", "*")
        params = []
        body = " ".join(m.group(3).split())
        if body and body != "void":
            for prm in body.split(","):
                toks = prm.replace("*", " * ").split()
                name = toks[-1]
                ctype = " ".join(toks[:-1]).replace(" *", "*")
                params.append((ctype, name))
        fns.append((m.group(2), ret, params))
    return fns


def rust_functions():
    text = open(FFI).read()
    block = text[text.index('extern "C" {'):]
    fns = []
    for m in re.finditer(r"pub fn (lh_\w+)\(([^)]*)\)(?:\s*->\s*([^;]+))?;", block):
        params = []
        if m.group(2).strip():
            for prm in m.group(2).split(","):
                name, ty = prm.split(":", 1)
                params.append((ty.strip(), name.strip()))
        fns.append((m.group(1), (m.group(3) or "()").strip(), params))
    return fns


def test_every_header_function_is_bound_with_matching_signature():
    cf, rf = c_functions(), rust_functions()
    assert len(cf) >= 100, len(cf)
    assert [f[0] for f in cf] == [f[0] for f in rf], "function sets or their order differ"
    assert len({f[0] for f in rf}) == len(rf), "a function is declared twice"
    for (name, cret, cparams), (_, rret, rparams) in zip(cf, rf):
        want_ret = "()" if cret == "void" else TYPE_MAP[cret]
        assert rret == want_ret, f"{name}: returns {rret}, header says {cret}"
        assert len(cparams) == len(rparams), f"{name}: {len(rparams)} arguments, header has {len(cparams)}"
        for (ctype, cname), (rtype, rname) in zip(cparams, rparams):
            assert rname.rstrip("_") == cname, f"{name}: argument {rname} vs {cname}"
            assert ctype in TYPE_MAP, f"{name}: no mapping for C type {ctype!r}"
            assert rtype == TYPE_MAP[ctype], f"{name}({cname}): {rtype}, header says {ctype}"


def test_enums_and_constants_agree():
    h = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    r = open(FFI).read()
    for body, ename in re.findall(r"typedef\s+enum\s+\w+\s*\{(.*?)\}\s*(\w+)\s*;", h, flags=re.S):
        for k, v in re.findall(r"(\w+)\s*=\s*(\d+)", body):
            if ename == "lh_status":
                assert re.search(rf"pub const {k}: c_int = {v};", r), k
            else:
                assert re.search(rf"pub enum {ename} \{{[^}}]*\b{k} = {v}\b", r), (ename, k)
    assert "pub const LH_TQ_SEED: u64 = 0x7459C0DE;" in r        # quant_cache.rs:30
    assert "pub const LH_DEFAULT_KV_BITS: c_int = 2;" in r        # quant_cache.rs:37


def test_library_exports_what_ffi_declares(pkg):
    lib = pkg.lib()
    missing = [f[0] for f in rust_functions() if not hasattr(lib, f[0])]
    assert not missing, missing


def test_ffi_is_up_to_date_with_the_header():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "local-hip", "gen_ffi.py"), "--check"], capture_output=True, text=True)
    assert out.returncode == 0, out.stderr


def test_build_script_uses_the_kernel_makefile():
    text = open(os.path.join(ROOT, "local-hip", "build.rs")).read()
    assert "local-ai_amd" in text and "csrc" in text and "rustc-link-lib=dylib=local_hip" in text
    mk = open(os.path.join(ROOT, "local-ai_amd", "csrc", "Makefile")).read()
    assert "OUT ?=" in mk and "BUILD ?=" in mk      # the two variables build.rs overrides
