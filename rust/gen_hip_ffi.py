#!/usr/bin/env python3
"""Writes rust/src/hip_ffi.rs from include/ag_hip.h: one `pub fn` per declared C function, in the
header's order, with the header's comment lines dropped.  Run it after the header changes;
tests/test_rust_shim.py checks (with its own parser) that the two files still agree."""
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "..", "include", "ag_hip.h")
OUT = os.path.join(HERE, "src", "hip_ffi.rs")

C_TO_RUST = {
    "ag_status_t": "AgStatus", "ag_stream_t": "AgStream", "int": "c_int", "long long": "c_longlong", "size_t": "usize",
    "float": "f32", "void": "()",
    "const float *": "*const f32", "float *": "*mut f32", "const float *const *": "*const *const f32",
    "float *const *": "*const *mut f32", "const size_t *": "*const usize",
    "void *": "*mut c_void", "const void *": "*const c_void", "const int *": "*const c_int", "int *": "*mut c_int",
    "uint8_t *": "*mut u8", "const uint8_t *": "*const u8", "const char *": "*const c_char",
}
RUST_KEYWORDS = {"type", "ref", "in", "fn", "mod", "move", "box", "loop", "match", "where", "use", "as", "self"}


def declarations(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = text[text.index('extern "C" {'):]
    for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b(ag_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        ret = " ".join(m.group(1).split())
        args = [] if m.group(3).strip() in ("", "void") else [" ".join(a.split()) for a in m.group(3).split(",")]
        yield ret, m.group(2), args


def split_arg(arg):
    m = re.match(r"(.*?)([A-Za-z_]\w*)$", arg)
    ctype, name = m.group(1).strip(), m.group(2)
    ctype = re.sub(r"\s*\*", " *", ctype).strip()
    ctype = ctype.replace("* const", "*const").replace("*const *", "*const *")
    return ctype, name


def rust_type(ctype):
    key = re.sub(r"\s+", " ", ctype).replace(" * ", " *").strip()
    key = key.replace("const float *const*", "const float *const *")
    return C_TO_RUST[key]


def main():
    lines = [
        "// Foreign declarations of libag_hip.so for the crate (to sit next to src/tensor_ops/blas_ffi.rs,",
        "// the reference's only other FFI: cblas_sgemm / cblas_dgemm through cblas-sys, blas_ffi.rs:1-15).",
        "// GENERATED from include/ag_hip.h by rust/gen_hip_ffi.py -- one `pub fn` per C function, same order.",
        "// UNCOMPILED in this repository: the image it was written in has no Rust toolchain.",
        "#![allow(clippy::too_many_arguments, non_snake_case)]",
        "use std::os::raw::{c_char, c_int, c_longlong, c_void};",
        "",
        "pub type AgStatus = c_int; // ag_status_t: 0 ok, 1..5 = op::OpError variants in order, 100 + n = hipError_t n",
        "pub type AgStream = *mut c_void; // hipStream_t",
        "",
        '#[link(name = "ag_hip")]',
        'extern "C" {',
    ]
    for ret, name, args in declarations(open(HEADER).read()):
        rargs = []
        for a in args:
            ctype, an = split_arg(a)
            if an in RUST_KEYWORDS:
                an += "_"
            rargs.append(f"{an}: {rust_type(ctype)}")
        rret = rust_type(re.sub(r"\s*\*", " *", ret))
        tail = "" if rret == "()" else f" -> {rret}"
        lines.append(f"    pub fn {name}({', '.join(rargs)}){tail};")
    lines += [
        "}",
        "",
        "/// ag_status_t -> the crate's OpError (src/op.rs:66-73); 1..5 are its variants in declaration order.",
        "pub fn to_op_error(st: AgStatus) -> crate::op::OpError {",
        "    let msg = unsafe { std::ffi::CStr::from_ptr(ag_last_error()) }.to_string_lossy().into_owned();",
        "    match st {",
        "        1 => crate::op::OpError::NdArrayError(msg, ndarray::ShapeError::from_kind(ndarray::ErrorKind::IncompatibleLayout)),",
        "        2 => crate::op::OpError::IncompatibleShape(msg),",
        "        3 => crate::op::OpError::TypeUnsupported(msg),",
        "        5 => crate::op::OpError::OutOfBounds(msg),",
        "        _ => crate::op::OpError::InvalidDims(msg), // 4, and 100 + hipError_t",
        "    }",
        "}",
        "",
        "/// `Ok(())` for AG_OK, the mapped OpError otherwise.",
        "pub fn check(st: AgStatus) -> Result<(), crate::op::OpError> {",
        "    if st == 0 { Ok(()) } else { Err(to_op_error(st)) }",
        "}",
        "",
    ]
    with open(OUT, "w") as f:
        f.write("\n".join(lines))


if __name__ == "__main__":
    main()
