"""Writes rust/src/ffi.rs, the Rust `extern "C"` block for every prototype of include/lumen_hip.h.

Usage: python rust/gen_ffi.py [--check]    (--check: exit 1 when the committed file is out of date)

The reference crate is Rust; this file is what a maintainer drops into it as src/ffi.rs (add `mod ffi;` and
link liblumen_hip.so from build.rs).
No Rust toolchain exists where this library is built, so the output is generated text, not compiled code."""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(os.path.dirname(HERE), "include", "lumen_hip.h")
OUT = os.path.join(HERE, "src", "ffi.rs")

SCALARS = {"int": "c_int", "float": "c_float", "double": "f64", "size_t": "usize", "int32_t": "i32", "uint16_t": "u16",
           "int64_t": "i64", "uint64_t": "u64", "char": "c_char", "void": "c_void"}
OPAQUE = ["lumen_ctx", "lumen_rope", "lumen_kv_cache", "lumen_llama"]
STRUCTS = {"lumen_llama_config", "lumen_sampling"}


def rust_type(ctype):
    t = ctype.strip()
    const = False
    stars = t.count("*")
    t = t.replace("*", " ").split()
    if t and t[0] == "const":
        const = True
        t = t[1:]
    if t and t[0] == "struct":
        t = t[1:]
    base = " ".join(t)
    if stars == 0:
        return SCALARS[base]
    inner = SCALARS.get(base, base)
    out = inner
    for level in range(stars):
        innermost = level == 0
        out = ("*const " if (const and innermost) else "*mut ") + out
    return out


def prototypes(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    text = re.sub(r"typedef struct \w* ?\{.*?\} \w+;", "", text, flags=re.S)
    for m in re.finditer(r"([\w\s\*]+?)\b(lumen_\w+)\s*\(([^;{}]*?)\)\s*;", text, flags=re.S):
        ret, name, args = m.group(1).strip(), m.group(2), " ".join(m.group(3).split())
        if ret.startswith("typedef") or not ret:
            continue
        params = []
        if args and args != "void":
            for a in args.split(","):
                a = a.strip()
                mm = re.match(r"(.*?)(\w+)$", a)
                params.append((mm.group(2), mm.group(1)))
        yield ret, name, params


def struct_fields(text, name):
    body = re.search(r"typedef struct (?:%s )?\{([^}]*)\} %s;" % (name, name), text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = []
    for decl in body.split(";"):
        decl = " ".join(decl.split())
        if not decl:
            continue
        first = decl.split(",")[0]
        ctype = first.rsplit(" ", 1)[0]
        names = [first.rsplit(" ", 1)[1]] + [n.strip() for n in decl.split(",")[1:]]
        for n in names:
            fields.append((n, rust_type(ctype)))
    return fields


def generate():
    text = open(HEADER).read()
    out = ["// Generated from include/lumen_hip.h by rust/gen_ffi.py -- do not edit.",
           "// Rust binding of liblumen_hip.so: src/ffi.rs + `mod ffi;` in the reference crate; link the library from build.rs.",
           "#![allow(non_camel_case_types, dead_code)]",
           "use std::os::raw::{c_char, c_float, c_int, c_void};", ""]
    for o in OPAQUE:
        out.append("#[repr(C)] pub struct %s { _private: [u8; 0] }" % o)
    out.append("")
    for sname in sorted(STRUCTS):
        out.append("#[repr(C)]\n#[derive(Clone, Copy, Debug)]\npub struct %s {" % sname)
        for n, t in struct_fields(text, sname):
            out.append("    pub %s: %s," % (n, t))
        out.append("}\n")
    for m in re.finditer(r"#define (LUMEN_\w+) (-?\d+)\b", text):
        out.append("pub const %s: c_int = %s;" % (m.group(1), m.group(2)))
    out.append("")
    out.append('extern "C" {')
    for ret, name, params in prototypes(text):
        sig = ", ".join("%s: %s" % (("r#%s" % n) if n in ("type", "match", "ref", "in") else n, rust_type(t)) for n, t in params)
        r = rust_type(ret)
        out.append("    pub fn %s(%s)%s;" % (name, sig, "" if ret == "void" else " -> " + r))
    out.append("}")
    out += ["", "/// status -> panic with the library's message: the reference's own error behaviour (Cargo.toml: panic = \"abort\")",
            "pub fn check(rc: c_int) {", "    if rc != 0 {",
            "        let msg = unsafe { std::ffi::CStr::from_ptr(lumen_last_error()) }.to_string_lossy().into_owned();",
            "        panic!(\"{msg}\");", "    }", "}", ""]
    return "\n".join(out)


if __name__ == "__main__":
    new = generate()
    if "--check" in sys.argv:
        old = open(OUT).read() if os.path.exists(OUT) else ""
        sys.exit(0 if old == new else 1)
    open(OUT, "w").write(new)
    print("wrote", OUT)
