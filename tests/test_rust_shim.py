"""The Rust half of the binding (rust/) cannot be compiled here -- there is no rustc -- so this checks
what a parser can: include/ag_hip.h and the `extern "C"` block of rust/src/hip_ffi.rs declare the
same functions with the same arity and C-compatible types, rust/build.rs compiles the sources
csrc/build.sh does, and rust/src/gpu_ops.rs implements `Op<f32>` for every operator of the path and
calls only declared functions with the declared number of arguments."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# C type (normalised) -> the Rust spellings that are ABI-compatible with it
COMPATIBLE = {
    "ag_status_t": {"AgStatus", "c_int", "i32"},
    "ag_stream_t": {"AgStream", "*mut c_void"},
    "int": {"c_int", "i32"},
    "long long": {"c_longlong", "i64"},
    "size_t": {"usize"},
    "float": {"f32"},
    "void": {"()"},
    "const float*": {"*const f32"},
    "float*": {"*mut f32"},
    "const float*const*": {"*const *const f32"},
    "float*const*": {"*const *mut f32"},
    "const size_t*": {"*const usize"},
    "void*": {"*mut c_void"},
    "const int*": {"*const c_int", "*const i32"},
    "uint8_t*": {"*mut u8"},
    "const uint8_t*": {"*const u8"},
    "const char*": {"*const c_char"},
}


def _norm_c(t):
    t = re.sub(r"\s+", " ", t).strip()
    return re.sub(r"\s*\*\s*", "*", t)


def c_prototypes():
    text = open(os.path.join(ROOT, "include", "ag_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = text[text.index('extern "C" {'):]
    protos = {}
    for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b(ag_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        ret, name, args = m.group(1), m.group(2), m.group(3).strip()
        types = []
        if args not in ("", "void"):
            for a in args.split(","):
                a = " ".join(a.split())
                types.append(_norm_c(re.match(r"(.*?)[A-Za-z_]\w*$", a).group(1)))
        protos[name] = (_norm_c(ret), types)
    return protos


def rust_prototypes():
    text = open(os.path.join(ROOT, "rust", "src", "hip_ffi.rs")).read()
    block = text[text.index('extern "C" {'):]
    block = block[:block.index("\n}\n")]
    protos = {}
    for m in re.finditer(r"pub fn (ag_[a-z0-9_]+)\(([^)]*)\)\s*(?:->\s*([^;]+))?;", block):
        name, args, ret = m.group(1), m.group(2).strip(), (m.group(3) or "()").strip()
        types = [a.split(":", 1)[1].strip() for a in args.split(",")] if args else []
        protos[name] = (ret, types)
    return protos


def test_every_c_function_is_declared_in_rust_with_compatible_types():
    c, r = c_prototypes(), rust_prototypes()
    assert len(c) >= 50
    assert sorted(c) == sorted(r), f"only in C: {sorted(set(c) - set(r))}; only in Rust: {sorted(set(r) - set(c))}"
    for name, (cret, cargs) in c.items():
        rret, rargs = r[name]
        assert rret in COMPATIBLE[cret], f"{name}: returns {cret} in C, {rret} in Rust"
        assert len(cargs) == len(rargs), f"{name}: {len(cargs)} arguments in C, {len(rargs)} in Rust"
        for i, (ct, rt) in enumerate(zip(cargs, rargs)):
            assert rt in COMPATIBLE[ct], f"{name}: argument {i} is {ct} in C, {rt} in Rust"


def test_rust_declarations_are_in_the_header_order_and_regenerate_identically():
    c = list(c_prototypes())
    r = list(rust_prototypes())
    assert c == r
    import importlib.util
    spec = importlib.util.spec_from_file_location("gen_hip_ffi", os.path.join(ROOT, "rust", "gen_hip_ffi.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    want = open(gen.OUT).read()
    gen.OUT = os.path.join(ROOT, "rust", "src", ".hip_ffi_check.rs")
    try:
        gen.main()
        assert open(gen.OUT).read() == want, "rust/src/hip_ffi.rs is stale: run rust/gen_hip_ffi.py"
    finally:
        if os.path.exists(gen.OUT):
            os.remove(gen.OUT)


def test_build_rs_compiles_the_sources_of_build_sh():
    sh = open(os.path.join(ROOT, "rust-autograd_amd", "csrc", "build.sh")).read()
    srcs = re.search(r"srcs=\(([^)]*)\)", sh).group(1).split()
    rs = open(os.path.join(ROOT, "rust", "build.rs")).read()
    listed = re.findall(r'"([a-z0-9_]+)"', rs[rs.index("const SOURCES"):rs.index("];")])
    assert sorted(listed) == sorted(s[:-4] for s in srcs)
    for s in srcs:
        assert os.path.exists(os.path.join(ROOT, "rust-autograd_amd", "csrc", s))
    for flag in ("--offload-arch=gfx950", "-packed-fp32-ops", "-ffp-contract=off"):
        assert flag in rs and flag in sh


def test_gpu_ops_implements_every_operator_and_calls_only_declared_functions():
    text = open(os.path.join(ROOT, "rust", "src", "gpu_ops.rs")).read()
    impls = set(re.findall(r"impl Op<f32> for (\w+)", text))
    assert impls == {"GpuConv2D", "GpuConv2DWithCols", "GpuConv2DFilterGrad", "GpuConv2DTranspose",
                     "GpuConv2DTransposeFilterGrad", "GpuMaxPool2D", "GpuMaxPool2DGrad", "GpuMaxPool2DGradGrad",
                     "GpuMatMul", "GpuBatchMatMul", "GpuReduceSumToScalar", "GpuReduceSum", "GpuReduceMean", "GpuAdamOp"}
    for name in impls:
        body = text[text.index(f"impl Op<f32> for {name}"):]
        body = body[:body.index("\n}\n")]
        assert "fn compute(" in body and "fn grad(" in body, name
    r = rust_prototypes()
    calls = re.findall(r"ffi::(ag_[a-z0-9_]+)\(", text)
    assert len(set(calls)) >= 18
    for m in re.finditer(r"ffi::(ag_[a-z0-9_]+)\(", text):
        name = m.group(1)
        assert name in r, f"gpu_ops.rs calls {name}, which hip_ffi.rs does not declare"
        # argument count of the call: split the balanced parenthesis at top-level commas
        depth, i, n_args, seen = 1, m.end(), 0, False
        while depth:
            ch = text[i]
            if ch in "([{":
                depth += 1
            elif ch in ")]}":
                depth -= 1
            elif ch == "," and depth == 1:
                n_args += 1
            if depth and not ch.isspace():
                seen = True
            i += 1
        n_args = n_args + 1 if seen else 0
        assert n_args == len(r[name][1]), f"{name}: called with {n_args} arguments, declared with {len(r[name][1])}"
