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


# What each operator's `grad` builds in the reference: (node built, its inputs, its back-prop inputs)
# in order, then which input gradients are Some.  Read off the reference's sources at the lines cited;
# the names are the reference's (the GPU twin of `X` is `GpuX`), the input expressions are normalised
# (`&`, whitespace and `ctx.` dropped).
REFERENCE_GRADS = {
    # conv_ops/conv2d.rs:556-586
    "Conv2D": ([("Conv2DTranspose", ["gy", "w"], []),
                ("Conv2DFilterGrad", ["cols", "gy", "w"], ["x", "gy"])], [True, True]),
    # conv_ops/conv2d.rs:599-628
    "Conv2DWithCols": ([("Conv2DTranspose", ["gy", "w"], []),
                        ("Conv2DFilterGrad", ["cols", "gy", "w"], ["y.get_backprop_input(0)", "gy"])], [True, True]),
    # conv_ops/conv2d.rs:746-775
    "Conv2DFilterGrad": ([("Conv2DTranspose", ["gy", "ggw"], []),
                          ("Conv2DWithCols", ["cols", "ggw"], ["y.get_backprop_input(0)", "ggw"])], [True, True]),
    # conv_ops/conv2d_transpose.rs:274-300
    "Conv2DTranspose": ([("Conv2D", ["gy", "w"], []),
                         ("Conv2DTransposeFilterGrad", ["gy", "x", "stop_gradient(w)"], [])], [True, True]),
    # conv_ops/conv2d_transpose.rs:453-479
    "Conv2DTransposeFilterGrad": ([("Conv2DTranspose", ["x", "gw"], []),
                                   ("Conv2D", ["gy", "gw"], [])], [True, True, False]),
    # conv_ops/max_pool2d.rs:229-242, :281-294, :333-336
    "MaxPool2D": ([("MaxPool2DGrad", ["gy", "indices"], [])], [True]),
    "MaxPool2DGrad": ([("MaxPool2DGradGrad", ["ggx", "argmax"], [])], [True, False]),
    "MaxPool2DGradGrad": ([], [False, False]),
    # dot_ops.rs:608-628, :697-717 (flags false/true then true/false, whatever the op's own flags)
    "MatMul": ([("MatMul{transpose_a:false,transpose_b:true}", ["gy", "input(1)"], []),
                ("MatMul{transpose_a:true,transpose_b:false}", ["input(0)", "gy"], [])], [True, True]),
    "BatchMatMul": ([("BatchMatMul{transpose_a:false,transpose_b:true}", ["gy", "input(1)"], []),
                     ("BatchMatMul{transpose_a:true,transpose_b:false}", ["input(0)", "gy"], [])], [True, True]),
    # reduction_ops.rs:130-136, :172-184, :217-238 (the CPU gradient ops serve: they are fills and broadcasts)
    "ReduceSumToScalar": ([("ReduceSumToScalarGrad", ["output_grad()", "shape(input(0))"], [])], [True]),
    "ReduceSum": ([("ReduceGradCommon", ["output_grad()", "shape(input(0))", "input(1)"], [])], [True, False]),
    "ReduceMean": ([("ReduceGradCommon", ["output_grad()", "shape(x)", "axes"], [])], [True, False]),
    # gradient_descent_ops/adam.rs:60-66
    "AdamOp": ([], [False] * 5),
}


def _grad_body(text, name):
    body = text[text.index(f"impl Op<f32> for {name} {{"):]
    body = body[:body.index("\n}\n")]
    return body[body.index("fn grad("):]


def _split_top(s):
    out, depth, cur = [], 0, ""
    for ch in s:
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur)
    return out


def _norm_expr(e):
    return re.sub(r"\s+", "", e).replace("&", "").replace("ctx.", "")


def _norm_op(op):
    op = re.sub(r"\s+", "", op)
    op = re.sub(r"^crate::tensor_ops::reduction_ops::", "", op)
    op = re.sub(r"\(self\.0\)$", "", op)           # the hyper-parameters travel unchanged
    if op.startswith("ReduceGradCommon"):
        assert "should_make_broadcast_dims:!self.keep_dims" in op and "sparse_axes:self.sparse_axes" in op
        op = "ReduceGradCommon"
    return re.sub(r"^Gpu", "", op)


def _built_nodes(body):
    """The nodes a `grad` body builds, in source order, from both spellings: `node(ctx, &[..], Op)` and
    `Tensor::builder(..).append_input(..)...build(Op)`."""
    found = []
    for m in re.finditer(r"\bnode\(ctx,\s*&\[([^\]]*)\],\s*", body):
        depth, i = 1, m.end()
        while depth:
            depth += {"(": 1, "{": 1, ")": -1, "}": -1}.get(body[i], 0)
            i += 1
        found.append((m.start(), _norm_op(body[m.end():i - 1]), [_norm_expr(e) for e in _split_top(m.group(1))], []))
    for m in re.finditer(r"Tensor::builder\(ctx\.graph\(\)\)", body):
        chain = body[m.end():]
        ins, bps, pos = [], [], 0
        while True:
            c = re.match(r"\s*\.(append_input|append_backprop_input|build)\(", chain[pos:])
            assert c, chain[pos:pos + 60]
            depth, i = 1, pos + c.end()
            while depth:
                depth += {"(": 1, "{": 1, ")": -1, "}": -1}.get(chain[i], 0)
                i += 1
            arg = chain[pos + c.end():i - 1]
            pos = i
            if c.group(1) == "append_input":
                expr, flag = _split_top(arg)
                assert flag.strip() == "false"
                ins.append(_norm_expr(expr))
            elif c.group(1) == "append_backprop_input":
                bps.append(_norm_expr(arg))
            else:
                found.append((m.start(), _norm_op(arg), ins, bps))
                break
    return [f[1:] for f in sorted(found)]


def test_every_gpu_grad_builds_the_nodes_the_reference_builds():
    text = open(os.path.join(ROOT, "rust", "src", "gpu_ops.rs")).read()
    for ref_name, (nodes, some) in REFERENCE_GRADS.items():
        body = _grad_body(text, "Gpu" + ref_name)
        got = [(op, ins, bps) for op, ins, bps in _built_nodes(body)]
        assert got == [(op, ins, bps) for op, ins, bps in nodes], f"Gpu{ref_name}::grad builds {got}"
        grads = re.findall(r"append_input_grad\((Some|None)", body)
        if ref_name == "AdamOp":
            assert "for _ in 0..5" in body and grads == ["None"]
        else:
            assert [g == "Some" for g in grads] == some, f"Gpu{ref_name}::grad returns {grads}"
    # the mean's gradient divides the broadcast by the product of the reduced extents (reduction_ops.rs:231-236)
    mean = _grad_body(text, "GpuReduceMean")
    assert "gather_common(shape(&x), &axes, 0)" in mean and "reduce_prod(reduced, &[0], false)" in mean and "broadcast / len" in mean
    assert set(REFERENCE_GRADS) == {n[3:] for n in re.findall(r"impl Op<f32> for (\w+)", text)}


def test_compute_bodies_move_arrays_only_through_device_io():
    """With device-resident storage the ops must not stage anything themselves: every input and output
    of every `compute` goes through the DeviceIo calls, whose two implementations (staging, resident)
    live in device.rs; the resident one relies on functions device_storage.rs defines."""
    ops = open(os.path.join(ROOT, "rust", "src", "gpu_ops.rs")).read()
    assert "upload(" not in ops and "download(" not in ops and ".assign(" not in ops and "input_mut(" not in ops
    for m in re.finditer(r"ctx\.input\((\d)\)", ops):
        line = ops[ops.rfind("\n", 0, m.start()):ops.find("\n", m.end())]
        fn = ops[:m.start()].rfind("fn ")
        in_grad = ops[fn:fn + 8] == "fn grad("
        assert in_grad or "axes_of(" in line, f"host read outside the axes list: {line.strip()}"
    dev = open(os.path.join(ROOT, "rust", "src", "device.rs")).read()
    trait = dev[dev.index("pub trait DeviceIo"):]
    trait = trait[:trait.index("\n}\n")]
    methods = re.findall(r"fn (\w+)\(", trait)
    assert methods == ["dev_in", "dev_in_mut", "dev_commit", "dev_out", "dev_out_shared"]
    assert dev.count("impl<'v> DeviceIo for ComputeContext<'v, f32>") == 2
    assert '#[cfg(not(feature = "device_storage"))]\nimpl<\'v> DeviceIo' in dev and '#[cfg(feature = "device_storage")]\nimpl<\'v> DeviceIo' in dev
    for used in set(re.findall(r"ctx\.(dev_\w+)\(", ops)):
        assert used in methods
    store = open(os.path.join(ROOT, "rust", "src", "device_storage.rs")).read()
    resident = dev[dev.rindex("impl<'v> DeviceIo for ComputeContext"):]
    for called in set(re.findall(r"self\.(\w+)\(", resident)):
        assert re.search(rf"pub fn {called}\(", store), f"device.rs relies on ComputeContext::{called}, which device_storage.rs does not define"
    for f in ("device_view", "device_view_mut", "sync_host_one", "take_to_host", "sync_host", "storage_get", "storage_take", "gather"):
        assert re.search(rf"fn {f}[<(]", store), f
