#!/usr/bin/env python3
"""Writes src/ffi.rs from include/nerva_hip_api.h: one #[repr(C)] struct per C struct (same field
order and widths) and one extern "C" declaration per entry point, so the Rust side of the boundary is
derived from the header the library is compiled against; and src/native_stubs.rs, the functions the
crate links instead of the library when hipcc is absent (every call fails with status -1 and
hip_error 100, like crates/nerva-cuda/src/native_stubs.rs:5-33).

    python crates/nerva-hip/generate_ffi.py            # rewrite src/ffi.rs
    python crates/nerva-hip/generate_ffi.py --check    # exit 1 when src/ffi.rs is out of date

(The reference's binding of its CUDA backend is written by hand:
crates/nerva-cuda/src/decode/hf_sequence/session/ffi.rs, .../hf_sequence/ffi.rs, projection/ffi.rs.)
"""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "..", "..", "include", "nerva_hip_api.h")
TARGET = os.path.join(HERE, "src", "ffi.rs")
STUBS = os.path.join(HERE, "src", "native_stubs.rs")

SCALARS = {"int32_t": "i32", "uint32_t": "u32", "uint64_t": "u64", "int64_t": "i64", "uint16_t": "u16",
           "uint8_t": "u8", "float": "f32", "double": "f64", "char": "c_char", "int": "c_int", "void": "c_void"}


def strip_comments(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def rust_type(base, stars, const, structs):
    if base in SCALARS:
        t = SCALARS[base]
    elif base in structs:
        t = base
    else:
        raise ValueError("unknown C type %r" % base)
    for i in range(stars):
        t = ("*const " if (const and i == 0) else "*mut ") + t
    return t


def parse(text):
    """-> (opaque struct names, [(struct, [(field, rust type)])], [(fn, ret, [(arg, rust type)])])"""
    opaque = re.findall(r"typedef struct (\w+) \1;", text)
    names = set(opaque) | set(re.findall(r"typedef struct (\w+) \{", text))
    structs = []
    for m in re.finditer(r"typedef struct (\w+) \{(.*?)\} \1;", text, flags=re.S):
        fields = []
        for decl in m.group(2).split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            const = decl.startswith("const ")
            decl = decl.replace("const ", "")
            base, rest = decl.split(" ", 1)
            for item in rest.split(","):
                item = item.strip()
                stars = item.count("*")
                ident = item.replace("*", "").strip()
                arr = re.match(r"(\w+)\[(\d+)\]$", ident)
                t = rust_type(base, stars, const, names)
                if arr:
                    ident, t = arr.group(1), "[%s; %s]" % (t, arr.group(2))
                fields.append((ident, t))
        structs.append((m.group(1), fields))
    functions = []
    for m in re.finditer(r"\b(int|uint64_t)\s+(nerva_hip_\w+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        args = []
        body = " ".join(m.group(3).split())
        if body != "void":
            for arg in body.split(","):
                arg = arg.strip()
                const = arg.startswith("const ")
                arg = arg.replace("const ", "")
                stars = arg.count("*")
                parts = arg.replace("*", " ").split()
                args.append((parts[-1], rust_type(parts[0], stars, const, names)))
        functions.append((m.group(2), SCALARS[m.group(1)], args))
    return opaque, structs, functions


def render():
    opaque, structs, functions = parse(strip_comments(open(HEADER).read()))
    out = ["//! The C ABI of libnerva_hip as Rust sees it. GENERATED from include/nerva_hip_api.h by",
           "//! generate_ffi.py - edit the header and regenerate; tests/test_rust_mirror_cpu.py fails when",
           "//! this file and the header disagree.",
           "#![allow(non_camel_case_types, non_snake_case, dead_code)]", "",
           "use std::os::raw::{c_char, c_int, c_void};", ""]
    for name in opaque:
        out += ["/// Opaque to callers: created by session_create, released by session_destroy.", "#[repr(C)]",
                "pub struct %s {" % name, "    _private: [u8; 0],", "}", ""]
    for name, fields in structs:
        out += ["#[repr(C)]", "#[derive(Copy, Clone)]", "pub struct %s {" % name]
        out += ["    pub %s: %s," % (("r#type" if f == "type" else f), t) for f, t in fields]
        out += ["}", ""]
    out += ['unsafe extern "C" {']
    for fn, ret, args in functions:
        out.append("    pub fn %s(%s) -> %s;" % (fn, ", ".join("%s: %s" % a for a in args), ret))
    out += ["}", ""]
    return "\n".join(out)


def render_stubs():
    opaque, structs, functions = parse(strip_comments(open(HEADER).read()))
    fields = {name: [f for f, _ in fs] for name, fs in structs}
    out = ["//! What the crate links when libnerva_hip is not built (no hipcc): every entry point fails the",
           "//! way the library itself fails without a device - status = -1, hip_error = 100 in results that",
           "//! carry them, null session handles, return value -1 (0 for size queries). GENERATED by",
           "//! generate_ffi.py.", "#![allow(unused_variables)]", "",
           "use std::os::raw::{c_int, c_void};", "", "use crate::ffi::*;", "",
           "const HIP_ERROR_NO_DEVICE: i32 = 100;", ""]
    for fn, ret, args in functions:
        body = []
        for name, t in args:
            if t.startswith("*mut *mut NervaHipHfDecodeSequenceSession"):
                body += ["    if !%s.is_null() {" % name, "        unsafe { %s.write(std::ptr::null_mut()) };" % name, "    }"]
            m = re.match(r"\*mut (NervaHip\w+)$", t)
            if m and fields.get(m.group(1), [])[:1] == ["status"]:
                body += ["    if !%s.is_null() {" % name, "        unsafe {", "            (*%s).status = -1;" % name]
                if "hip_error" in fields[m.group(1)]:
                    body.append("            (*%s).hip_error = HIP_ERROR_NO_DEVICE;" % name)
                body += ["        }", "    }"]
            if name == "hip_error" and t == "*mut i32":
                body += ["    if !hip_error.is_null() {", "        unsafe { hip_error.write(HIP_ERROR_NO_DEVICE) };", "    }"]
        body.append("    0" if ret == "u64" else "    -1")
        out += ["#[unsafe(no_mangle)]",
                'pub extern "C" fn %s(%s) -> %s {' % (fn, ", ".join("%s: %s" % a for a in args), ret)] + body + ["}", ""]
    return "\n".join(out)


if __name__ == "__main__":
    outputs = ((TARGET, render()), (STUBS, render_stubs()))
    if "--check" in sys.argv:
        sys.exit(0 if all(os.path.exists(p) and open(p).read() == t for p, t in outputs) else 1)
    for path, text in outputs:
        with open(path, "w") as f:
            f.write(text)
        print("wrote", os.path.relpath(path))
