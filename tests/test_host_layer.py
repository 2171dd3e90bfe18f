"""CPU-side tests of the host operator layer (libag_host.so): the library loads, its exported
symbols are exactly what include/ag_host.h declares and what the ctypes table binds, and graph
construction / gradient-graph structure follow the reference (no kernel runs without a GPU:
graphs here are built from placeholders only and never evaluated)."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def G():
    from __graft_entry__ import load_package

    load_package()
    import rust_autograd_amd.graph as graph

    graph.lib()
    return graph


def header_functions():
    text = open(os.path.join(ROOT, "include", "ag_host.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(agh_[a-z0-9_]+)\s*\(", text))


def test_exports_match_header_and_bindings(G):
    out = subprocess.run(["nm", "-D", "--defined-only", G.host_library_path()], capture_output=True, text=True,
                         check=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T agh_" in line}
    declared = header_functions()
    assert declared == exported
    assert declared == set(G.PROTOTYPES)


def test_host_library_does_not_link_the_oracle(G):
    out = subprocess.run(["ldd", G.host_library_path()], capture_output=True, text=True, check=True).stdout
    assert "libag_hip.so" in out and "oracle" not in out and "openblas" not in out.lower()


def small_graph(G):
    env = G.VariableEnvironment()
    c = env.context()
    x = c.placeholder("x", [-1, 1, 8, 8])
    w = c.placeholder("w", [4, 1, 3, 3])
    return env, c, x, w


def test_conv2d_builds_a_two_output_node_with_selector(G):
    # conv2d() returns nth_tensor(Conv2D, 0) in the reference too (src/tensor_ops/mod.rs:2397-2423)
    env, c, x, w = small_graph(G)
    y = c.conv2d(x, w, 1, 1)
    assert y.op_name in ("Conv2D", "NthTensor")
    assert y.topo_rank >= 1
    assert x.topo_rank == 0 and w.topo_rank == 0


def test_grad_graph_uses_the_reference_ops(G):
    env, c, x, w = small_graph(G)
    y = c.conv2d(x, w, 1, 1)
    p = c.max_pool2d(c.relu(y), 2, 0, 2)
    before = c.num_nodes
    gx, gw = c.grad([c.sum_all(p)], [x, w])
    names = {c._t(i).op_name for i in range(before, c.num_nodes)}
    # Conv2D::grad builds Conv2DTranspose and Conv2DFilterGrad (conv2d.rs:219-247); MaxPool2D::grad
    # builds MaxPool2DGrad (max_pool2d.rs:229-242); ReLU::grad builds its mask op.
    assert {"Conv2DTranspose", "Conv2DFilterGrad", "MaxPool2DGrad"} <= names
    assert gx.op_name == "Conv2DTranspose" and gw.op_name == "Conv2DFilterGrad"


def test_grad_of_unreachable_input_is_zeros_like(G):
    # tensor_ops::grad substitutes zeros for an x the loss does not depend on
    env, c, x, w = small_graph(G)
    (g,) = c.grad([c.sum_all(c.relu(x))], [w])
    assert g.op_name == "Zeros"


def test_second_order_graph_builds(G):
    env, c, x, w = small_graph(G)
    y = c.conv2d(x, w, 1, 1)
    (gw,) = c.grad([c.sum_all(y)], [w])
    before = c.num_nodes
    (ggx,) = c.grad([c.sum_all(gw)], [x])
    names = {c._t(i).op_name for i in range(before, c.num_nodes)}
    # Conv2DFilterGrad::grad differentiates through Conv2DTranspose / Conv2DWithCols style ops
    assert names & {"Conv2DTranspose", "Conv2DWithCols", "Conv2DTransposeFilterGrad", "Conv2D"}
    assert ggx.id >= before


def test_topo_rank_is_one_more_than_the_deepest_input(G):
    env, c, x, w = small_graph(G)
    a = c.relu(x)
    b = c.relu(a)
    s = c.add(a, b)
    assert (a.topo_rank, b.topo_rank, s.topo_rank) == (1, 2, 3)


def test_the_sum_behind_a_fused_relu_is_on_the_backprop_path(G):
    # relu(a + b) is one AddReLU node over a and b whose back-prop input is the AddOp node: the sum must rank
    # below it and receive greater(z, 0) * gy (activation_ops.rs:154-167), not zeros
    env, c, x, w = small_graph(G)
    y = c.placeholder("y", [-1, 1, 8, 8])
    z = c.add(x, y)
    r = c.relu(z)
    assert r.op_name == "AddReLU" and r.num_inputs == 2 and r.topo_rank == z.topo_rank + 1
    gz, gx = c.grad([c.sum_all(r)], [z, x])
    assert gz.op_name == "ReLUGrad"
    assert gx.op_name == "MaybeReduceSum"
    # 0-dimensional operands keep the two nodes
    assert c.relu(c.add(c.scalar(1.0), c.scalar(2.0))).op_name == "ReLU"


def test_bad_handles_panic_with_a_message(G):
    env, c, x, w = small_graph(G)
    with pytest.raises(G.Panic, match="out of range"):
        c._t(G.lib().agh_relu(c._h, 12345))
    with pytest.raises(G.Panic, match="not found"):
        c.variable("missing")
    with pytest.raises(G.Panic):
        c.add_n([])
