"""CPU-side checks of the C-ABI boundary: the library loads, exports every symbol
include/lumen_hip.h declares, and (with no GPU in this process) refuses to compute
with a status instead of crashing or silently falling back."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "lumen_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lumen_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    from lumen_amd import _lib
    names = declared_symbols()
    assert len(names) >= 40
    assert set(names) == set(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    from lumen_amd import _lib
    assert os.path.exists(_lib.LIB_PATH)
    raw = C.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(raw, name), name
    assert b"gfx950" in _lib.lib.lumen_version()


def test_no_gpu_means_status_not_fallback():
    from lumen_amd import _lib
    h = C.c_void_p()
    rc = _lib.lib.lumen_ctx_create(0, C.byref(h))
    if rc == _lib.OK:  # running on a GPU box: nothing to check here
        _lib.lib.lumen_ctx_destroy(h)
        pytest.skip("a GPU is present")
    assert rc == _lib.ERR_NO_DEVICE and not h.value
    assert _lib.lib.lumen_last_error()
    with pytest.raises(_lib.LumenError):
        _lib.check(rc)
    # null handles are rejected, not dereferenced
    assert _lib.lib.lumen_gemv_f32(None, None, None, None, 4, 4) == _lib.ERR_INVALID
    assert _lib.lib.lumen_llama_forward(None, None, 1, None, 0) == _lib.ERR_INVALID


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "lumen_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".hpp", ".cpp")) or f == "Makefile":
                text = open(os.path.join(dirpath, f), errors="replace").read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)


def _header_without_comments():
    text = open(os.path.join(ROOT, "include", "lumen_hip.h")).read()
    return re.sub(r"/\*.*?\*/", "", text, flags=re.S)


def _split_args(arglist):
    arglist = " ".join(arglist.split())
    return [] if arglist in ("", "void") else [a.strip() for a in arglist.split(",")]


def _header_facts():
    """Prototypes (name -> parameter declarations), struct fields and integer constants of the header, parsed here
    -- not with the generator's code."""
    text = _header_without_comments()
    structs = {}
    for m in re.finditer(r"typedef struct\s*\w*\s*\{([^}]*)\}\s*(\w+)\s*;", text, flags=re.S):
        fields = []
        for decl in m.group(1).split(";"):
            decl = " ".join(decl.split())
            if decl:
                ctype, first = decl.split(",")[0].rsplit(" ", 1)
                for n in [first] + [x.strip() for x in decl.split(",")[1:]]:
                    fields.append((n.lstrip("*"), ctype.strip()))
        structs[m.group(2)] = fields
    body = re.sub(r"typedef struct\s*\w*\s*\{[^}]*\}\s*\w+\s*;", "", text, flags=re.S)
    protos = {m.group(1): _split_args(m.group(2))
              for m in re.finditer(r"\b(lumen_[a-z0-9_]+)\s*\(([^;{}()]*)\)\s*;", body)}
    consts = {m.group(1): int(m.group(2)) for m in re.finditer(r"^\s*#define\s+(LUMEN_\w+)\s+(-?\d+)\b", text, flags=re.M)}
    return protos, structs, consts


def test_rust_binding_is_in_step_with_the_header():
    """rust/src/ffi.rs is generated from the header: the committed file must be what the generator writes now, and
    -- checked with a parse of its own, against the header and against the ctypes table -- it must declare every
    function with the same number of parameters, pointers where the header has pointers, every struct with the
    same fields in the same order, and every integer constant with the same value."""
    import subprocess
    import sys
    rc = subprocess.run([sys.executable, os.path.join(ROOT, "rust", "gen_ffi.py"), "--check"]).returncode
    assert rc == 0, "run python rust/gen_ffi.py"
    from lumen_amd import _lib
    rs = open(os.path.join(ROOT, "rust", "src", "ffi.rs")).read()
    protos, structs, consts = _header_facts()
    assert set(protos) == set(_lib.SIGNATURES) and len(protos) >= 60
    rs_fns = {m.group(1): _split_args(m.group(2)) for m in re.finditer(r"pub fn (lumen_\w+)\(([^)]*)\)", rs)}
    assert set(rs_fns) == set(protos)
    for name, cargs in protos.items():
        rargs = rs_fns[name]
        assert len(rargs) == len(cargs) == len(_lib.SIGNATURES[name][1]), name
        for ca, ra, pa in zip(cargs, rargs, _lib.SIGNATURES[name][1]):
            rtype = ra.split(":", 1)[1].strip()
            assert ("*" in ca) == rtype.startswith("*"), (name, ca, ra)          # pointer <-> pointer
            assert rtype.count("*") == ca.count("*"), (name, ca, ra)             # same depth
            if "*" in ca:
                assert ("const" in ca.split("*")[0].split()) == rtype.startswith("*const"), (name, ca, ra)
                assert pa in (C.c_void_p, C.c_char_p) or issubclass(pa, C._Pointer), (name, ca, pa)
            else:
                scalar = {"int": C.c_int, "float": C.c_float, "size_t": C.c_size_t, "int64_t": C.c_int64,
                          "uint64_t": C.c_uint64, "double": C.c_double}[ca.rsplit(" ", 1)[0].strip()]
                assert pa is scalar, (name, ca, pa)
    rs_structs = {m.group(1): [tuple(x.strip() for x in f.split(":")) for f in re.findall(r"pub (\w+: [^,]+),", m.group(2))]
                  for m in re.finditer(r"pub struct (\w+) \{\n(.*?)\n\}", rs, flags=re.S)}
    assert len(structs) >= 2
    for sname, fields in structs.items():
        assert [n for n, _ in fields] == [n for n, _ in rs_structs[sname]], sname
        for (n, ctype), (_, rtype) in zip(fields, rs_structs[sname]):
            assert rtype == {"int": "c_int", "float": "c_float", "uint64_t": "u64", "int64_t": "i64"}[ctype], (sname, n)
    rs_consts = {m.group(1): int(m.group(2)) for m in re.finditer(r"pub const (LUMEN_\w+): c_int = (-?\d+);", rs)}
    assert rs_consts == consts and len(consts) >= 15
    # the hand-written part of the crate-side sources uses only what the binding declares
    gpu = open(os.path.join(ROOT, "rust", "src", "llama_gpu.rs")).read()
    for used in set(re.findall(r"(?<![\w:])ffi::(\w+)", gpu)):
        assert used in rs_fns or used in rs_consts or used in rs_structs or used in ("check", "lumen_ctx", "lumen_llama"), used
    for f in ("build.rs", "Cargo.toml.fragment"):
        assert os.path.exists(os.path.join(ROOT, "rust", f))


def test_gate_up_kernel_of_the_committed_counters_is_the_one_the_dispatch_picks():
    """bench.py quotes roofline.traffic from profiles/decode_gateup_gemv_traffic.json only for the kernel instance
    named there.  That name must be what the library's dispatch picks for the headline shape's gate|up product
    ([11264, 2048] f32, RMSNorm prologue, SwiGLU epilogue, 256 compute units): lumen_gemv_kernel_name reads the same
    decision function launch_gemv launches from, and needs no GPU."""
    import json
    from lumen_amd import _lib
    t = json.load(open(os.path.join(ROOT, "profiles", "decode_gateup_gemv_traffic.json")))
    picked = _lib.gemv_kernel_name(256, 11264, 2048, False, True, _lib.GEMV_EPI_SWIGLU)
    assert t["kernel"] == picked
    assert re.fullmatch(r"gemv_kernel<false, 2, 1, 2, \d, (true|false)>", picked)
    src = open(os.path.join(ROOT, "bench.py")).read()
    assert "gemv_kernel<" not in src  # bench.py prints the recorded name, it holds no kernel string of its own
    assert "measured_traffic(gu_kernel)" in src and 't["kernel"] != kernel' in src
    # other products of the step, as a guard on the decision function itself
    assert _lib.gemv_kernel_name(256, 2048, 5632, False, False, _lib.GEMV_EPI_RESIDUAL) == "gemv_kernel<false, 1, 0, 1, 4, false>"
    assert _lib.gemv_kernel_name(256, 32000, 2048, False, True, _lib.GEMV_EPI_ARGMAX) == "gemv_kernel<false, 2, 1, 3, 1, true>"
    assert _lib.gemv_kernel_name(256, 2048, 2047, False, False, _lib.GEMV_EPI_STORE) == "gemv_generic_kernel<false>"
