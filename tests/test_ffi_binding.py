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
    "int*": "*mut c_int",
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


# ---- the safe layer: local-hip/src/{kernels,error,buffer,batch,context}.rs --------------------------------------------
KERNELS_RS = os.path.join(ROOT, "local-hip", "src", "kernels.rs")
SAFE_TYPES = {"const lh_buffer*": "&Buffer", "lh_buffer*": "&Buffer", "const lh_buffer* const*": "&[&Buffer]",
              "lh_buffer* const*": "&[&Buffer]", "const uint32_t*": "&[u32]", "uint32_t": "u32", "uint64_t": "u64",
              "size_t": "usize", "float": "f32", "int": "c_int", "lh_quant": "ffi::lh_quant", "lh_dtype": "ffi::lh_dtype"}


def safe_methods():
    """[(method, [(name, type)], raw function called, [argument expressions])] parsed from kernels.rs."""
    text = open(KERNELS_RS).read()
    out = []
    for m in re.finditer(r"pub fn (\w+)\(&self, ([^)]*)\) -> Result<\(\)> \{(.*?)\n    \}", text, flags=re.S):
        params = [tuple(s.strip() for s in prm.split(":", 1)) for prm in m.group(2).split(", ")]
        call = re.search(r"ffi::(lh_\w+)\((.*?)\) \}\)", m.group(3), flags=re.S)
        out.append((m.group(1), params, call.group(1), [a.strip() for a in call.group(2).split(", ")]))
    return out


def test_safe_layer_methods_follow_the_header():
    """Every dispatch operation of the header (first parameter the batch or the context, the rest buffers, buffer arrays
    and scalars) has one `Kernels` method named as the header function less `lh_`, with the header's parameter names in the
    header's order and types that correspond, and the method hands them to that raw function in that order."""
    header = {f[0]: f for f in c_functions()}
    methods = safe_methods()
    assert len(methods) >= 60, len(methods)
    wrapped = set()
    for method, params, raw, args in methods:
        assert raw == "lh_" + method, (method, raw)
        _, cret, cparams = header[raw]
        assert cret == "int"
        wrapped.add(raw)
        assert len(params) == len(cparams) == len(args), method
        first_c = cparams[0][0]
        assert params[0] == (("batch", "&mut CommandBatch") if first_c == "lh_batch*" else ("ctx", "&Context")), method
        assert args[0] == params[0][0] + ".as_ptr()"
        for (pname, ptype), (ctype, cname), arg in zip(params[1:], cparams[1:], args[1:]):
            assert pname.rstrip("_") == cname, f"{method}: {pname} vs {cname}"
            assert ptype == SAFE_TYPES[ctype], f"{method}({cname}): {ptype} for {ctype}"
            want = {"&Buffer": f"{pname}.as_ptr()", "&[&Buffer]": f"{pname}_raw.as_ptr()", "&[u32]": f"{pname}.as_ptr()"}.get(ptype, pname)
            assert arg == want, f"{method}: passes {arg} for {cname}"
    # nothing that is a dispatch operation was left out
    for name, cret, cparams in header.values():
        is_op = bool(cret == "int" and cparams and cparams[0][0] in ("lh_batch*", "lh_context*")
                 and not name.startswith(("lh_context_", "lh_buffer_", "lh_batch_", "lh_event_", "lh_graph_"))
                 and all(t in SAFE_TYPES for t, _ in cparams[1:]))
        assert (name in wrapped) == is_op, name


def test_safe_layer_argument_order_of_the_reference():
    """Three methods whose parameter lists were read off the reference (local-metal/src/kernels.rs:4819-4834, 5176-5193,
    5434-5452; kept here as data): the generated methods take exactly these parameters in exactly this order."""
    want = {
        "encode_kv_turboquant_into": ["batch", "input", "levels", "signs", "packed", "norms", "head_dim", "n_kv_heads",
                                      "num_tokens", "bits", "position", "ring_capacity"],
        "flash_attention_tq_into": ["batch", "rq", "k_codes", "k_norms", "v_codes", "v_norms", "levels", "out", "head_dim",
                                    "kv_len", "current_pos", "num_q_heads", "num_kv_heads", "window", "bits", "ring_capacity"],
        "flash_attention_tq_batched_into": ["batch", "rq", "k_codes", "k_norms", "v_codes", "v_norms", "levels", "out",
                                            "positions", "head_dim", "lane_capacity", "num_q_heads", "num_kv_heads", "window",
                                            "bits", "n_lanes", "ring_capacity"],
    }
    have = {m: [p[0] for p in params] for m, params, _, _ in safe_methods()}
    for method, names in want.items():
        assert have[method] == names, method


def test_safe_layer_is_up_to_date_and_complete():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "local-hip", "gen_safe.py"), "--check"], capture_output=True, text=True)
    assert out.returncode == 0, out.stderr
    src = os.path.join(ROOT, "local-hip", "src")
    lib = open(os.path.join(src, "lib.rs")).read()
    for mod in ("batch", "buffer", "context", "error", "ffi", "kernels"):
        assert os.path.exists(os.path.join(src, mod + ".rs")), mod
        assert f"pub mod {mod};" in lib, mod
    err = open(os.path.join(src, "error.rs")).read()
    for variant in ("NoDevice", "NoCommandQueue", "BufferAllocation", "LibraryCreation", "PipelineCreation", "ShaderNotFound",
                    "CommandBuffer", "InvalidArgument", "Io"):          # local-metal/src/error.rs:1-32
        assert re.search(rf"\b{variant}\b", err), variant
    for code in ("LH_ERR_NO_DEVICE", "LH_ERR_NO_COMMAND_QUEUE", "LH_ERR_BUFFER_ALLOCATION", "LH_ERR_LIBRARY_CREATION",
                 "LH_ERR_PIPELINE_CREATION", "LH_ERR_SHADER_NOT_FOUND", "LH_ERR_COMMAND_BUFFER", "LH_ERR_IO"):
        assert f"ffi::{code} =>" in err, code
    # every raw function the hand-written modules call exists in ffi.rs with that many arguments
    raw = {f[0]: len(f[2]) for f in rust_functions()}
    for mod in ("batch", "buffer", "context", "error", "lib"):
        text = open(os.path.join(src, mod + ".rs")).read()
        for m in re.finditer(r"ffi::(lh_\w+)\(", text):
            name = m.group(1)
            assert name in raw, (mod, name)
            depth, n, i, seen = 1, 0, m.end(), False
            while depth:                      # walk to the matching parenthesis, counting top-level commas
                ch = text[i]
                depth += ch in "(["
                depth -= ch in ")]"
                seen = seen or (depth >= 1 and not ch.isspace())
                n += ch == "," and depth == 1
                i += 1
            n = n + 1 if seen else 0
            assert n == raw[name], (mod, name, n, raw[name])
