"""GPU tests of the host operator layer: the graphs the reference's examples and tests build
(conv block, small CNN with Adam, matmul / batch_matmul, transposed and dilated convolutions,
second-order gradients) are built through libag_host.so, evaluated on the GPU and compared with the
CPU oracle run stage by stage on the same inputs.

Tolerance for floating point: |got - want| <= 1e-5 + 1e-4 * |want|; contractions: 1e-5 + 2e-5 * the
magnitude their rounding errors scale with, and the literal bound on 99 % of the elements (the
kernels themselves are held to the f64 bars of tests/bars.py in test_gpu_parity.py); integer-valued results
(argmax-driven scatter positions, shapes, the Adam step counter) must be exact.
"""
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def say(msg):
    print(f"[graph] {msg}", flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def G():
    import torch

    assert torch.cuda.is_available(), "these tests need the MI355X"
    from __graft_entry__ import load_package

    load_package()
    import rust_autograd_amd.graph as graph

    graph.lib()
    return graph


def assert_close(got, want, what, rtol=None, atol=1e-5, scale=None):
    """Against the f32 oracle run stage by stage.  Without `scale`: the literal bound
    1e-5 + 1e-4*|want| on every element.  With `scale` (the magnitude rounding errors of the
    contraction behind `want` scale with): atol + 2e-5 * scale on every element -- two f32 results of
    the same contraction differ by a few units of roundoff of that magnitude, never by 1e-4 of it --
    and the literal bound on 99 % of the elements."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} != {want.shape}"
    if rtol is None:
        rtol = 1e-4 if scale is None else 2e-5
    bound = atol + rtol * (np.abs(want) if scale is None else scale)
    err = np.abs(got - want)
    bad = err > bound
    if scale is not None and err.size:
        say(f"{what}: worst err {float(err.max()):.3e}, err/scale {float((err / np.maximum(scale, 1e-300)).max()):.3e}, "
            f"literal {100.0 * float((err <= 1e-5 + 1e-4 * np.abs(want)).mean()):.3f} %")
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.size} outside tolerance, worst {float((err / bound).max()):.2f}x"
    if scale is not None and err.size:
        assert float((err <= 1e-5 + 1e-4 * np.abs(want)).mean()) >= 0.99, f"{what}: fewer than 99 % within 1e-5 + 1e-4|want|"


def glorot(rng, shape):
    fan_in = int(np.prod(shape[1:]))
    fan_out = shape[0] * int(np.prod(shape[2:])) if len(shape) > 2 else shape[0]
    if len(shape) == 2:
        fan_in, fan_out = shape
    sc = np.sqrt(6.0 / (fan_in + fan_out))
    return rng.uniform(-sc, sc, shape).astype(np.float32)


# ------------------------------------------------------------------------------- config 1
def test_config1_through_the_graph(G, orc, rng):
    B = 64
    xv = rng.random((B, 1, 28, 28), dtype=np.float32)
    wv = glorot(rng, (32, 1, 3, 3))
    env = G.VariableEnvironment()
    wid = env.set("w", wv)
    c = env.context()
    x = c.placeholder("x", [-1, 1, 28, 28])
    w = c.variable(wid)
    y = c.conv2d(x, w, 1, 1)
    p = c.max_pool2d(c.relu(y), 2, 0, 2)
    loss = c.reduce_sum(p, [0, 1, 2, 3])
    gx, gw = c.grad([loss], [x, w])
    say("config 1 eval")
    yv, pv, lv, gxv, gwv = c.eval([y, p, loss, gx, gw], {"x": xv})

    oy, ocols = orc.conv2d_fwd(xv, wv, 1, 1, 1)
    assert_close(yv, oy, "y")
    orl = orc.relu(yv)  # discrete stages are checked on the GPU's own conv output
    op, oam, _ = orc.maxpool2d_fwd(orl, 2, 0, 2)
    assert np.array_equal(pv, op)
    assert_close(lv, orc.reduce_sum(op, [0, 1, 2, 3]), "loss")
    ogr, _ = orc.maxpool2d_bwd(np.ones_like(op), oam, orl.shape)
    ogy = orc.relu_grad(yv, ogr)
    assert_close(gwv, orc.conv2d_filter_grad(ocols, ogy, wv.shape), "gw", scale=np.abs(gwv).max())
    assert_close(gxv, orc.conv2d_transpose(ogy, wv, 1, 1, 1), "gx")
    assert gxv.shape == xv.shape and gwv.shape == wv.shape


# ------------------------------------------------------------------------------- config 2
class OracleCNN:
    """The small CNN of examples/cnn_mnist.rs, forward and backward, stage by stage on the oracle."""

    def __init__(self, orc, params):
        self.o = orc
        self.p = {k: v.copy() for k, v in params.items()}

    def step_grads(self, x, labels, pre1=None, pre2=None):
        """`pre1`, `pre2`: the GPU's own inputs of the two ReLUs.  The ReLU masks and the pooling
        indices are then taken from them, as in the config-1 test: with about three million
        activations per step one of them lies within rounding of zero more often than not, and a
        different decision there moves one filter's gradient by a whole term."""
        o, p = self.o, self.p
        y1, cols1 = o.conv2d_fwd(x, p["w1"], 1, 1, 1)
        z1 = o.add_bias(y1.reshape(y1.shape[0], -1), p["b1"].reshape(-1)).reshape(y1.shape)
        if pre1 is not None:
            assert_close(pre1, z1, "first ReLU input")
            z1 = pre1
        r1 = o.relu(z1)
        p1, am1, _ = o.maxpool2d_fwd(r1, 2, 0, 2)
        y2, cols2 = o.conv2d_fwd(p1, p["w2"], 1, 1, 1)
        z2 = o.add_bias(y2.reshape(y2.shape[0], -1), p["b2"].reshape(-1)).reshape(y2.shape)
        if pre2 is not None:
            assert_close(pre2, z2, "second ReLU input")
            z2 = pre2
        r2 = o.relu(z2)
        p2, am2, _ = o.maxpool2d_fwd(r2, 2, 0, 2)
        flat = p2.reshape(p2.shape[0], -1)
        logits = o.add_bias(o.matmul(flat, p["w3"]), p["b3"].reshape(-1))
        per_row, lsm = o.sparse_softmax_xent(logits, labels)
        loss = o.reduce_mean(per_row, [0])
        n = per_row.shape[0]
        g_rows = np.full((n, 1), np.float32(1.0) / np.float32(n), dtype=np.float32)
        g_logits = o.sparse_softmax_xent_grad(lsm, labels, g_rows)
        g = {}
        g["b3"] = g_logits.sum(axis=0, dtype=np.float64).astype(np.float32).reshape(p["b3"].shape)
        g["w3"] = o.matmul(flat, g_logits, ta=True)
        g_flat = o.matmul(g_logits, p["w3"], tb=True)
        g_r2, _ = o.maxpool2d_bwd(g_flat.reshape(p2.shape), am2, r2.shape)
        g_z2 = o.relu_grad(z2, g_r2)
        g["b2"] = g_z2.sum(axis=0, dtype=np.float64).astype(np.float32).reshape(p["b2"].shape)
        g["w2"] = o.conv2d_filter_grad(cols2, g_z2, p["w2"].shape)
        g_p1 = o.conv2d_transpose(g_z2, p["w2"], 1, 1, 1)
        g_r1, _ = o.maxpool2d_bwd(g_p1, am1, r1.shape)
        g_z1 = o.relu_grad(z1, g_r1)
        g["b1"] = g_z1.sum(axis=0, dtype=np.float64).astype(np.float32).reshape(p["b1"].shape)
        g["w1"] = o.conv2d_filter_grad(cols1, g_z1, p["w1"].shape)
        return loss, logits, g


def cnn_params(rng):
    return {
        "w1": glorot(rng, (32, 1, 3, 3)),
        "w2": glorot(rng, (64, 32, 3, 3)),
        "w3": glorot(rng, (64 * 7 * 7, 10)),
        "b1": np.zeros((1, 32, 28, 28), np.float32),
        "b2": np.zeros((1, 64, 14, 14), np.float32),
        "b3": np.zeros((1, 10), np.float32),
    }


def build_cnn(G, env, c):
    v = {k: c.variable(k) for k in ("w1", "w2", "w3", "b1", "b2", "b3")}
    x = c.placeholder("x", [-1, 1, 28, 28])
    t = c.placeholder("y", [-1, 1])
    pre1 = c.conv2d(x, v["w1"], 1, 1) + v["b1"]
    z2 = c.max_pool2d(c.relu(pre1), 2, 0, 2)
    pre2 = c.conv2d(z2, v["w2"], 1, 1) + v["b2"]
    z4 = c.max_pool2d(c.relu(pre2), 2, 0, 2)
    z5 = c.reshape(z4, [-1, 64 * 7 * 7])
    logits = c.matmul(z5, v["w3"]) + v["b3"]
    loss = c.sparse_softmax_cross_entropy(logits, t)
    return v, logits, loss, (pre1, pre2)


def test_config2_training_steps_with_adam(G, orc, rng):
    B = 128
    params = cnn_params(rng)
    env = G.VariableEnvironment()
    ids = {k: env.set(k, a) for k, a in params.items()}
    names = ["w1", "w2", "w3", "b1", "b2", "b3"]
    adam = G.Adam(env, [ids[k] for k in names], alpha=1e-3)
    ref = OracleCNN(orc, params)
    m = {k: np.zeros_like(a) for k, a in params.items()}
    vv = {k: np.zeros_like(a) for k, a in params.items()}
    tt = {k: np.ones(1, np.float32) for k in params}
    solid_so_far = {k: np.ones(a.shape, bool) for k, a in params.items()}

    for step in range(3):
        xv = rng.random((B, 1, 28, 28), dtype=np.float32)
        lab = rng.integers(0, 10, (B, 1)).astype(np.float32)
        c = env.context()  # a fresh graph per step, as `env.run(|ctx| ...)` in the example's loop
        v, logits, loss, pre = build_cnn(G, env, c)
        mean_loss = c.reduce_mean(loss, [0], False)
        grads = c.grad([mean_loss], [v[k] for k in names])
        say(f"config 2 step {step}: grads")
        out = c.eval([mean_loss, logits] + grads + list(pre), {"x": xv, "y": lab})
        oloss, ologits, og = ref.step_grads(xv, lab, out[-2], out[-1])
        out = out[:-2]
        assert_close(out[1], ologits, f"logits step {step}", scale=1.0)
        assert_close(out[0], oloss, f"loss step {step}")
        for k, gv in zip(names, out[2:]):
            scale = np.abs(og[k]).max()
            assert_close(gv, og[k], f"grad {k} step {step}", scale=scale, atol=1e-7)
        say(f"config 2 step {step}: update")
        adam.update([v[k] for k in names], grads, c, {"x": xv, "y": lab})
        for k in names:
            orc.adam(ref.p[k], og[k], m[k], vv[k], tt[k], alpha=1e-3)
            # The update's size is alpha whatever the gradient's, so compare on that scale; where
            # the gradient is a near-total cancellation its relative error, and with it the
            # update's, is unbounded: those elements only have to stay within the step size.
            got, want = env.array(ids[k]), ref.p[k]
            solid_so_far[k] &= np.abs(og[k]) >= 1e-3 * np.abs(og[k]).max()
            solid = solid_so_far[k]
            assert_close(got[solid], want[solid], f"param {k} after step {step}", scale=1e-3, rtol=1e-4, atol=1e-7)
            assert np.abs(got - want).max() <= 2.1e-3
        # Every step is checked from identical state: Adam moves an element by about alpha whatever the
        # size of its gradient, so an element whose gradient is rounding noise can move the other way,
        # and a ReLU input that close to zero then switches for the whole batch in the next step.
        for k in names:
            ref.p[k][...] = env.array(ids[k])
            m[k][...] = env.array(env.find(f"{ids[k]}m", "adam"))
            vv[k][...] = env.array(env.find(f"{ids[k]}v", "adam"))
            solid_so_far[k][...] = True
    # optimizer state lives in the environment under the optimizer's namespace (adam.rs:66-89)
    for k in names:
        tid = env.find(f"{ids[k]}t", "adam")
        assert tid is not None and env.array(tid).reshape(-1)[0] == 4.0
        assert env.find(f"{ids[k]}m", "adam") is not None and env.find(f"{ids[k]}v", "adam") is not None


def test_config2_free_running_loss_trajectory(G, orc, rng):
    """Four training steps on one batch with nothing re-synchronised in between: the device runs its own graph with
    its own Adam state, the oracle its own stages (its own ReLU masks and pooling indices) with the oracle's Adam.
    Single elements may part ways (an activation within rounding of zero, a gradient that is rounding noise moving
    its parameter by alpha the other way); the loss, a mean over the batch, must follow the oracle's trajectory to
    1e-3 relative, and must fall."""
    B = 128
    params = cnn_params(rng)
    env = G.VariableEnvironment()
    ids = {k: env.set(k, a) for k, a in params.items()}
    names = ["w1", "w2", "w3", "b1", "b2", "b3"]
    adam = G.Adam(env, [ids[k] for k in names], alpha=1e-3)
    ref = OracleCNN(orc, params)
    m = {k: np.zeros_like(a) for k, a in params.items()}
    vv = {k: np.zeros_like(a) for k, a in params.items()}
    tt = {k: np.ones(1, np.float32) for k in params}
    xv = rng.random((B, 1, 28, 28), dtype=np.float32)
    lab = rng.integers(0, 10, (B, 1)).astype(np.float32)
    got, want = [], []
    for step in range(4):
        c = env.context()
        v, logits, loss, _ = build_cnn(G, env, c)
        mean_loss = c.reduce_mean(loss, [0], False)
        grads = c.grad([mean_loss], [v[k] for k in names])
        say(f"config 2 free-running step {step}")
        update = adam.get_update_op([v[k] for k in names], grads, c)
        # the loss is requested last, so it is visited first: it is the loss before this step's update
        got.append(float(np.asarray(c.eval([update, mean_loss], {"x": xv, "y": lab})[1]).reshape(-1)[0]))
        oloss, _, og = ref.step_grads(xv, lab)
        want.append(float(np.asarray(oloss).reshape(-1)[0]))
        for k in names:
            orc.adam(ref.p[k], og[k], m[k], vv[k], tt[k], alpha=1e-3)
    say(f"losses {got} oracle {want}")
    for step, (a, b) in enumerate(zip(got, want)):
        assert abs(a - b) <= 1e-3 * abs(b), f"step {step}: loss {a} against the oracle's {b}"
    assert got[-1] < got[0] and want[-1] < want[0]
    for k in names:   # the parameters themselves stay within a few steps' worth of alpha of the oracle's
        assert np.abs(env.array(ids[k]) - ref.p[k]).max() <= 4 * 2.1e-3


def test_grad_helper_returns_every_variable_of_the_namespace(G, rng):
    env = G.VariableEnvironment()
    env.set("a", rng.random((4, 3), dtype=np.float32))
    env.set("b", rng.random((1, 3), dtype=np.float32))
    c = env.context()
    x = c.placeholder("x", [-1, 4])
    loss = c.sum_all(c.matmul(x, c.variable("a")) + c.variable("b"))
    vs, gs = c.grad_helper([loss])
    assert len(vs) == 2 and len(gs) == 2
    xv = rng.random((5, 4), dtype=np.float32)
    ga, gb = c.eval(gs, {"x": xv})
    got = {tuple(ga.shape): ga, tuple(gb.shape): gb}
    assert_close(got[(4, 3)], np.repeat(xv.sum(axis=0)[:, None], 3, axis=1), "d/da")
    assert_close(got[(1, 3)], np.full((1, 3), 5.0), "d/db")


# ------------------------------------------------------------------------------- config 3 (reduced)
@pytest.mark.parametrize("shape", [((96, 200), (200, 72)), ((1, 17), (17, 1))])
def test_matmul_and_its_gradients(G, orc, rng, shape):
    av, bv = (rng.standard_normal(s).astype(np.float32) for s in shape)
    env = G.VariableEnvironment()
    c = env.context()
    a, b = c.placeholder("a", list(shape[0])), c.placeholder("b", list(shape[1]))
    z = c.matmul(a, b)
    ga, gb = c.grad([c.sum_all(z)], [a, b])
    say(f"matmul {shape}")
    zv, gav, gbv = c.eval([z, ga, gb], {"a": av, "b": bv})
    k = shape[0][1]
    assert_close(zv, orc.matmul(av, bv), "z", scale=np.sqrt(k))
    ones = np.ones_like(zv)
    assert_close(gav, orc.matmul(ones, bv, tb=True), "ga", scale=np.abs(bv).sum(axis=1)[None, :] + 0 * gav)
    assert_close(gbv, orc.matmul(av, ones, ta=True), "gb", scale=np.abs(av).sum(axis=0)[:, None] + 0 * gbv)


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_batch_matmul_and_its_gradients(G, orc, rng, ta, tb):
    Bt, M, K, N = 6, 40, 56, 24
    av = rng.standard_normal((Bt, K, M) if ta else (Bt, M, K)).astype(np.float32)
    bv = rng.standard_normal((Bt, N, K) if tb else (Bt, K, N)).astype(np.float32)
    env = G.VariableEnvironment()
    c = env.context()
    a, b = c.placeholder("a", list(av.shape)), c.placeholder("b", list(bv.shape))
    z = c.batch_matmul(a, b, ta, tb)
    ga, gb = c.grad([c.sum_all(z)], [a, b])
    say(f"batch_matmul ta={ta} tb={tb}")
    zv, gav, gbv = c.eval([z, ga, gb], {"a": av, "b": bv})
    assert_close(zv, orc.batch_matmul(av, bv, ta, tb), "z", scale=np.sqrt(K))
    # BatchMatMul::grad builds batch_matmul(gy, b^T) and batch_matmul(a^T, gy) whatever the op's own
    # transpose flags are (dot_ops.rs:697-717), so like the reference the gradients are those of
    # sum(z) only for untransposed operands; with a flag set they are shape errors or differently
    # shaped products, exactly as there.
    ones = np.ones_like(zv)
    for got, args, what in ((gav, (ones, bv, False, True), "ga"), (gbv, (av, ones, True, False), "gb")):
        try:
            want = orc.batch_matmul(*args)
        except Exception:
            assert isinstance(got, G.OpError), what
            continue
        assert_close(got, want, what, scale=np.sqrt(max(M, N)))
    if not ta and not tb:
        gA = np.repeat(bv.astype(np.float64).sum(axis=2)[:, None, :], M, axis=1)
        gB = np.repeat(av.astype(np.float64).sum(axis=1)[:, :, None], N, axis=2)
        assert_close(gav, gA, "ga analytic", scale=np.sqrt(N))
        assert_close(gbv, gB, "gb analytic", scale=np.sqrt(M))


# ------------------------------------------------------------------------------- configs 4 / 5 (reduced)
@pytest.mark.parametrize("H,pad,stride,dil,k", [(14, 1, 1, 1, 3), (16, 1, 2, 1, 3), (14, 2, 1, 2, 3), (15, 0, 2, 1, 2)])
def test_conv2d_gradients_every_geometry(G, orc, rng, H, pad, stride, dil, k):
    B, Cin, Cout = 3, 5, 7
    xv = rng.standard_normal((B, Cin, H, H)).astype(np.float32)
    wv = glorot(rng, (Cout, Cin, k, k))
    env = G.VariableEnvironment()
    c = env.context()
    x, w = c.placeholder("x", list(xv.shape)), c.placeholder("w", list(wv.shape))
    y = c.dilated_conv2d(x, w, pad, stride, dil)
    gyv = None
    gx, gw = c.grad([c.sum_all(c.mul(y, y))], [x, w])
    say(f"conv grads H={H} pad={pad} stride={stride} dil={dil} k={k}")
    yv, gxv, gwv = c.eval([y, gx, gw], {"x": xv, "w": wv})
    oy, ocols = orc.conv2d_fwd(xv, wv, pad, stride, dil)
    assert_close(yv, oy, "y", scale=1.0)
    gyv = (2 * yv).astype(np.float32)
    assert_close(gwv, orc.conv2d_filter_grad(ocols, gyv, wv.shape), "gw", scale=np.abs(gwv).max())
    # the gradient has x's own extent, also where the transposed-convolution size formula would
    # come out one short (stride 2 on an even extent)
    assert gxv.shape == xv.shape
    assert_close(gxv, orc.conv2d_transpose(gyv, wv, pad, stride, dil, out_hw=(H, H)), "gx", scale=np.abs(gxv).max())
    # what the reference itself returns (extent rebuilt from gy, conv2d_transpose.rs:55-56) is the
    # top-left crop of that gradient
    ref_like = orc.conv2d_transpose(gyv, wv, pad, stride, dil)
    h = ref_like.shape[2]
    assert h <= H
    assert_close(gxv[:, :, :h, :h], ref_like, "gx crop", scale=np.abs(gxv).max())


def test_conv2d_transpose_upsampling_and_gradients(G, orc, rng):
    B, Cin, Cout, H = 4, 12, 6, 7
    xv = rng.standard_normal((B, Cin, H, H)).astype(np.float32)
    wv = rng.uniform(-0.1, 0.1, (Cin, Cout, 4, 4)).astype(np.float32)
    env = G.VariableEnvironment()
    c = env.context()
    x, w = c.placeholder("x", list(xv.shape)), c.placeholder("w", list(wv.shape))
    y = c.conv2d_transpose(x, w, 1, 2)
    gx, gw = c.grad([c.sum_all(c.mul(y, y))], [x, w])
    say("conv2d_transpose 4x4 stride 2")
    yv, gxv, gwv = c.eval([y, gx, gw], {"x": xv, "w": wv})
    assert yv.shape == (B, Cout, 14, 14)
    assert_close(yv, orc.conv2d_transpose(xv, wv, 1, 2, 1), "y", scale=1.0)
    gyv = (2 * yv).astype(np.float32)
    # d/dx of a transposed convolution is the forward convolution of gy with the same filter
    ogx, _ = orc.conv2d_fwd(gyv, wv, 1, 2, 1)
    assert_close(gxv, ogx, "gx", scale=np.abs(ogx).max())
    assert_close(gwv, orc.conv2d_transpose_filter_grad(xv, gyv, wv.shape, 1, 2, 1), "gw", scale=np.abs(gwv).max())


def test_max_pool_gradient_and_second_order(G, orc, rng):
    xv = rng.standard_normal((2, 3, 9, 9)).astype(np.float32)
    env = G.VariableEnvironment()
    c = env.context()
    x = c.placeholder("x", list(xv.shape))
    y = c.max_pool2d(x, 3, 0, 2)
    (gx,) = c.grad([c.sum_all(c.mul(y, y))], [x])
    (ggx,) = c.grad([c.sum_all(c.mul(gx, gx))], [x])  # runs MaxPool2DGradGrad (max_pool2d.rs:297-337)
    say("max pool second order")
    yv, gxv, ggxv = c.eval([y, gx, ggx], {"x": xv})
    oy, oam, _ = orc.maxpool2d_fwd(xv, 3, 0, 2)
    assert np.array_equal(yv, oy)
    ogx, _ = orc.maxpool2d_bwd((2 * oy).astype(np.float32), oam, xv.shape)
    assert np.array_equal(gxv, ogx)
    assert ggxv.shape == xv.shape and np.isfinite(ggxv).all()


def test_second_order_conv_filter_grad_wrt_input(G, orc, rng):
    # sum over the filter gradient of sum(conv(x, w)) is linear in x: its gradient is the
    # transposed convolution of an all-ones gy with an all-ones filter.
    xv = rng.standard_normal((2, 3, 8, 8)).astype(np.float32)
    wv = glorot(rng, (4, 3, 3, 3))
    env = G.VariableEnvironment()
    c = env.context()
    x, w = c.placeholder("x", list(xv.shape)), c.placeholder("w", list(wv.shape))
    y = c.conv2d(x, w, 1, 1)
    (gw,) = c.grad([c.sum_all(y)], [w])
    (ggx,) = c.grad([c.sum_all(gw)], [x])
    say("second order conv")
    gwv, ggxv = c.eval([gw, ggx], {"x": xv, "w": wv})
    _, ocols = orc.conv2d_fwd(xv, wv, 1, 1, 1)
    ones_gy = np.ones((2, 4, 8, 8), np.float32)
    assert_close(gwv, orc.conv2d_filter_grad(ocols, ones_gy, wv.shape), "gw", scale=np.abs(gwv).max())
    assert_close(ggxv, orc.conv2d_transpose(ones_gy, np.ones_like(wv), 1, 1, 1), "ggx")


@pytest.mark.parametrize("axes,keep", [([0], False), ([1], True), ([0, 2], False), ([-1], False)])
def test_reduce_ops_and_gradients(G, orc, rng, axes, keep):
    xv = rng.standard_normal((6, 5, 4)).astype(np.float32)
    env = G.VariableEnvironment()
    c = env.context()
    x = c.placeholder("x", list(xv.shape))
    s, m = c.reduce_sum(x, axes, keep), c.reduce_mean(x, axes, keep)
    (gs,) = c.grad([c.sum_all(c.mul(s, s))], [x])
    (gm,) = c.grad([c.sum_all(m)], [x])
    sv, mv, gsv, gmv = c.eval([s, m, gs, gm], {"x": xv})
    assert np.array_equal(sv, orc.reduce_sum(xv, axes, keep))
    assert np.array_equal(mv, orc.reduce_mean(xv, axes, keep))
    ax = [a % 3 for a in axes]
    assert_close(gsv, np.broadcast_to(2 * xv.sum(axis=tuple(ax), keepdims=True), xv.shape), "d sum^2", atol=1e-4)
    count = int(np.prod([xv.shape[a] for a in ax]))
    assert_close(gmv, np.full(xv.shape, 1.0 / count), "d mean")


def test_finite_difference_check_of_a_conv_block(G, rng):
    # the reference's own way of testing gradients (src/test_helper.rs:11-94): central differences
    xv = rng.standard_normal((1, 2, 6, 6)).astype(np.float32)
    wv = rng.standard_normal((3, 2, 3, 3)).astype(np.float32)
    env = G.VariableEnvironment()
    wid = env.set("w", wv)
    c = env.context()
    x = c.placeholder("x", list(xv.shape))
    loss = c.sum_all(c.mul(c.conv2d(x, c.variable(wid), 1, 1), c.conv2d(x, c.variable(wid), 1, 1)))
    (gw,) = c.grad([loss], [c.variable(wid)])
    gwv = c.eval([gw], {"x": xv})[0]
    eps = 1e-2
    for idx in [(0, 0, 0, 0), (2, 1, 1, 1), (1, 0, 2, 1)]:
        vals = []
        for sgn in (+1, -1):
            wp = wv.copy()
            wp[idx] += sgn * eps
            env2 = G.VariableEnvironment()
            w2 = env2.set("w", wp)
            c2 = env2.context()
            x2 = c2.placeholder("x", list(xv.shape))
            y2 = c2.conv2d(x2, c2.variable(w2), 1, 1)
            vals.append(float(c2.eval([c2.sum_all(c2.mul(y2, y2))], {"x": xv})[0]))
        numeric = (vals[0] - vals[1]) / (2 * eps)
        assert abs(numeric - gwv[idx]) <= 2e-2 * max(1.0, abs(numeric)), (idx, numeric, gwv[idx])


# ------------------------------------------------------------------------------- error behaviour
def test_op_errors_come_back_as_results_and_misuse_panics(G, rng):
    env = G.VariableEnvironment()
    c = env.context()
    a, b = c.placeholder("a", [-1, -1]), c.placeholder("b", [-1, -1])
    z = c.matmul(a, b)
    ok = c.relu(a)
    av, bv = rng.random((3, 4), dtype=np.float32), rng.random((5, 2), dtype=np.float32)
    r = c.eval([z, ok], {"a": av, "b": bv})
    # evaluation.rs:341-360: a failed op yields Err for that tensor, the others still evaluate
    assert isinstance(r[0], G.OpError) and r[0].kind == "IncompatibleShape"
    assert np.array_equal(r[1], av)
    with pytest.raises(G.Panic, match="[Pp]laceholder"):
        c.eval([z], {"a": av})
    x4 = c.placeholder("x4", [-1, 3, 8, 8])
    w4 = c.placeholder("w4", [4, 2, 3, 3])
    r = c.eval([c.conv2d(x4, w4, 1, 1)], {"x4": rng.random((1, 3, 8, 8), dtype=np.float32),
                                         "w4": rng.random((4, 2, 3, 3), dtype=np.float32)})
    assert isinstance(r[0], G.OpError)


def test_variables_are_shared_between_contexts_and_updated_in_place(G, orc, rng):
    env = G.VariableEnvironment()
    wv = rng.random((8, 8), dtype=np.float32) + 2.0
    wid = env.set("w", wv)
    adam = G.Adam(env, [wid], alpha=0.5)
    p, m, v, t = wv.copy(), np.zeros_like(wv), np.zeros_like(wv), np.ones(1, np.float32)
    for step in range(2):
        c = env.context()
        w = c.variable(wid)
        (g,) = c.grad([c.sum_all(c.mul(w, w))], [w])
        adam.update([w], [g], c)
        orc.adam(p, (p + p).astype(np.float32), m, v, t, alpha=0.5)
        assert_close(env.array(wid), p, f"Adam step {step}")
    # with a constant-sign gradient Adam moves every element by about alpha per step
    assert np.abs(env.array(wid) - (wv - 1.0)).max() < 0.05


def test_feeds_and_read_backs_of_any_size_cross_the_staging_ring_intact(G, rng):
    """Host arrays travel through a 16 MiB page-locked ring: many small feeds wrap it several times, a feed larger
    than the ring takes the synchronous path, and the caller's buffer may be overwritten as soon as eval returns."""
    env = G.VariableEnvironment()
    c = env.context()
    x = c.placeholder("x", [-1, 1024])
    y = c.relu(x)
    buf = np.empty((300, 1024), np.float32)                     # 1.2 MB per feed: the ring wraps every 13 feeds
    for i in range(40):
        buf[:] = rng.random((300, 1024), dtype=np.float32) + 0.5
        want = buf.copy()
        (got,) = c.eval([y], {"x": buf})
        buf[:] = -1.0                                           # reuse of the caller's buffer must not reach the device
        assert np.array_equal(got, want), f"feed {i}"
    big = rng.random((5000, 1024), dtype=np.float32) + 0.5      # 20.5 MB > the ring
    (got,) = c.eval([y], {"x": big})
    assert np.array_equal(got, big)
    wid = env.set("w", big)                                     # variables are uploaded the same way
    assert np.array_equal(env.array(wid), big)


def test_relu_of_a_sum_is_one_node_with_the_values_and_gradients_of_two(G, orc, rng):
    """relu(a + b) is built as one fused node over a and b.  Its value, and the gradients that reach a and the
    broadcast b through it, must have exactly the bits of the unfused graph (relu applied to the sum through an
    identity, which hides the AddOp from the fusion)."""
    env = G.VariableEnvironment()
    av = rng.standard_normal((6, 5, 4, 4)).astype(np.float32)
    bv = rng.standard_normal((1, 5, 1, 1)).astype(np.float32)
    aid, bid = env.set("a", av), env.set("b", bv)
    c = env.context()
    a, b = c.variable(aid), c.variable(bid)
    fused = c.relu(a + b)
    assert fused.op_name == "AddReLU" and fused.num_inputs == 2
    plain = c.relu(c.reshape(a + b, [6, 5, 4, 4]))
    assert plain.op_name == "ReLU"
    wts = c.placeholder("wts", [6, 5, 4, 4])
    gf = c.grad([c.sum_all(c.mul(fused, wts))], [a, b])
    gp = c.grad([c.sum_all(c.mul(plain, wts))], [a, b])
    wv = rng.standard_normal((6, 5, 4, 4)).astype(np.float32)
    yf, yp, gfa, gfb, gpa, gpb = c.eval([fused, plain, *gf, *gp], {"wts": wv})
    want = np.maximum(av + bv, 0)
    assert np.array_equal(yf, want) and np.array_equal(yp, want)
    assert np.array_equal(gfa.view(np.uint32), gpa.view(np.uint32)) and np.array_equal(gfa, wv * (av + bv > 0))
    assert gfb.shape == (1, 5, 1, 1) and np.array_equal(gfb.view(np.uint32), gpb.view(np.uint32))


def test_the_sum_inside_a_fused_relu_stays_differentiable(G, rng):
    """relu(z) with z = a + b is one fused node over a and b, but z itself must stay on the back-propagation path:
    the gradient with respect to z is greater(z, 0) * gy (activation_ops.rs:154-167), also when z feeds a second
    consumer, and with respect to a and b it is the bits of the unfused graph."""
    env = G.VariableEnvironment()
    av = rng.standard_normal((6, 5, 4, 4)).astype(np.float32)
    bv = rng.standard_normal((1, 5, 1, 1)).astype(np.float32)
    wv = rng.standard_normal((6, 5, 4, 4)).astype(np.float32)
    aid, bid = env.set("a", av), env.set("b", bv)
    c = env.context()
    a, b = c.variable(aid), c.variable(bid)
    wts = c.placeholder("wts", [6, 5, 4, 4])
    z = a + b
    fused = c.relu(z)
    assert fused.op_name == "AddReLU"
    zp = a + b
    plain = c.relu(c.reshape(zp, [6, 5, 4, 4]))
    assert plain.op_name == "ReLU"
    (gz,) = c.grad([c.sum_all(c.mul(fused, wts))], [z])
    (gzp,) = c.grad([c.sum_all(c.mul(plain, wts))], [zp])
    (gzd,) = c.grad_with_default([fused], [z], [wts])
    # z with a second consumer: both contributions must meet in its gradient, and reach a and b
    both = c.sum_all(c.mul(fused, wts)) + c.sum_all(c.mul(z, wts))
    gz2, ga2, gb2 = c.grad([both], [z, a, b])
    bothp = c.sum_all(c.mul(plain, wts)) + c.sum_all(c.mul(zp, wts))
    gzp2, gap2, gbp2 = c.grad([bothp], [zp, a, b])
    say("gradient with respect to the sum inside relu(a + b)")
    r = c.eval([gz, gzp, gzd, gz2, ga2, gb2, gzp2, gap2, gbp2], {"wts": wv})
    mask = (av + bv > 0)
    assert np.array_equal(r[0], wv * mask) and np.array_equal(r[0].view(np.uint32), r[1].view(np.uint32))
    assert np.array_equal(r[2], wv * mask)
    assert np.array_equal(r[3], wv * mask + wv)
    for got, want in zip(r[3:6], r[6:9]):
        assert got.shape == want.shape and np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # operands of rank 0 keep the two nodes (the fused kernel takes ranks 1..8), with the same value
    s = c.relu(c.scalar(-2.0) + c.scalar(0.5))
    t = c.relu(c.scalar(2.0) + c.scalar(0.5))
    assert s.op_name == "ReLU"
    sv, tv = c.eval([s, t], {})
    assert sv.shape == () and float(sv) == 0.0 and float(tv) == 2.5


@pytest.mark.parametrize("H,size,stride", [(14, 2, 2), (28, 2, 2), (13, 3, 2), (9, 2, 1)])
def test_relu_gradient_behind_a_pooling_is_one_node_with_the_pooling_gradient(G, rng, H, size, stride):
    """max_pool2d(relu(x)): the gradient that reaches x is built as one node (the pooling's backward with the ReLU's
    mask applied as it stores) instead of MaxPool2DGrad followed by ReLUGrad.  Values and second-order gradients
    must have the bits of the two-node form, which a reshape between the ReLU and the pooling forces."""
    B, C = 3, 5
    xv = rng.standard_normal((B, C, H, H)).astype(np.float32)
    env = G.VariableEnvironment()
    c = env.context()
    x = c.placeholder("x", [B, C, H, H])
    OH = (H - size) // stride + 1
    wts = c.placeholder("wts", [B, C, OH, OH])
    fused_y = c.max_pool2d(c.relu(x), size, 0, stride)
    plain_y = c.max_pool2d(c.reshape(c.relu(x), [B, C, H, H]), size, 0, stride)
    (gf,) = c.grad([c.sum_all(c.mul(fused_y, wts))], [x])
    (gp,) = c.grad([c.sum_all(c.mul(plain_y, wts))], [x])
    assert gf.op_name == "MaxPool2DGradReLU" and gp.op_name == "ReLUGrad"
    # second order: the gradient of <gx, v> with respect to the weights of the first-order loss
    v = c.placeholder("v", [B, C, H, H])
    (hf,) = c.grad([c.sum_all(c.mul(gf, v))], [wts])
    (hp,) = c.grad([c.sum_all(c.mul(gp, v))], [wts])
    wv = rng.standard_normal((B, C, OH, OH)).astype(np.float32)
    vv = rng.standard_normal((B, C, H, H)).astype(np.float32)
    say(f"relu gradient fused into the pooling backward H={H} size={size} stride={stride}")
    a, b, ha, hb = c.eval([gf, gp, hf, hp], {"x": xv, "wts": wv, "v": vv})
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.array_equal(ha.view(np.uint32), hb.view(np.uint32))
    assert np.count_nonzero(a) > 0 and np.all(a[xv <= 0] == 0)


@pytest.mark.parametrize("with_bias", [False, True])
def test_relu_in_front_of_a_2x2_pooling_is_evaluated_with_it(G, rng, with_bias):
    """max_pool2d(relu(x), 2, 0, 2) and max_pool2d(relu(x + b), 2, 0, 2): when the evaluator reaches the pooling and its
    input has not been computed, the two nodes run as one launch (the graph keeps both nodes; src/evaluation.rs runs
    every node on its own).  Values, the ReLU's own result when it is asked for as well, and the gradients must have
    the bits of the nodes evaluated in turn, whichever of them the walk reaches first."""
    B, C, H = 3, 5, 12
    xv = rng.standard_normal((B, C, H, H)).astype(np.float32)
    bv = rng.standard_normal((1, C, 1, 1)).astype(np.float32)
    wv = rng.standard_normal((B, C, H // 2, H // 2)).astype(np.float32)
    env = G.VariableEnvironment()
    xid, bid = env.set("x", xv), env.set("b", bv)

    def graph(c, split):
        x, b = c.variable(xid), c.variable(bid)
        r = c.relu(x + b) if with_bias else c.relu(x)
        src = c.reshape(r, [B, C, H, H]) if split else r     # the reshape keeps the pooling away from the ReLU
        y = c.max_pool2d(src, 2, 0, 2)
        wts = c.placeholder("wts", [B, C, H // 2, H // 2])
        grads = c.grad([c.sum_all(c.mul(y, wts))], [x, b] if with_bias else [x])
        return r, y, grads

    say(f"relu evaluated together with the pooling behind it, bias: {with_bias}")
    results = {}
    for split in (False, True):
        for order in ("y first", "r first", "grads only"):
            c = env.context()
            r, y, grads = graph(c, split)
            wanted = {"y first": [y, r] + grads, "r first": [r, y] + grads, "grads only": grads}[order]
            out = c.eval(wanted, {"wts": wv})
            assert c.fused_pairs == (0 if split else 1), (split, order, c.fused_pairs)
            named = dict(zip(["y", "r"] if order == "y first" else ["r", "y"], out[:2])) if order != "grads only" else {}
            named.update({f"g{i}": g for i, g in enumerate(out[-len(grads):])})
            results[(split, order)] = named
    ref = results[(True, "y first")]
    want_r = np.maximum(xv + bv, 0) if with_bias else np.maximum(xv, 0)
    assert np.array_equal(ref["r"], want_r)
    for key, named in results.items():
        for name, arr in named.items():
            assert arr.shape == ref[name].shape and np.array_equal(arr.view(np.uint32), ref[name].view(np.uint32)), (key, name)
    # odd planes do not fuse and still evaluate
    c = env.context()
    x5 = c.placeholder("x5", [2, 3, 5, 7])
    (y5,) = c.eval([c.max_pool2d(c.relu(x5), 2, 0, 2)], {"x5": rng.standard_normal((2, 3, 5, 7)).astype(np.float32)})
    assert y5.shape == (2, 3, 2, 3) and c.fused_pairs == 0


def test_constant_gradients_through_reductions_are_one_fill_with_the_bits_of_the_chain(G, rng):
    """The seed of a back-propagation is a constant, and so is what the reductions at the end of a loss broadcast it
    to: those nodes are built as one FilledLike node (a single fill at evaluation) whose value goes through the
    divisions of the mean reductions in their order.  Against the unfolded chain, which a seed fed at run time
    forces (same bits), and against the arithmetic done by hand."""
    B, D = 3, 7
    xv = rng.standard_normal((B, D)).astype(np.float32)
    env = G.VariableEnvironment()
    c = env.context()
    x = c.placeholder("x", [B, D])
    seed = c.placeholder("seed", [1])
    loss = c.reduce_mean(c.reduce_mean(x, [1], True), [0], False)        # [1]
    (g_folded,) = c.grad([loss], [x])
    (g_chain,) = c.grad_with_default([loss], [x], [seed])
    assert g_folded.op_name == "FilledLike" and g_chain.op_name == "ReduceGradCommon"
    sq = c.reduce_mean(c.mul(x, x), [0, 1], True)                         # data-dependent below the reduction
    (h_folded,) = c.grad([sq], [x])
    (h_chain,) = c.grad_with_default([sq], [x], [c.placeholder("seed0", [1, 1])])
    say("constant gradients folded into one fill")
    a, b, hf, hc, total = c.eval([g_folded, g_chain, h_folded, h_chain, c.sum_all(x)],
                                 {"x": xv, "seed": np.ones(1, np.float32), "seed0": np.ones((1, 1), np.float32)})
    want = np.float32(np.float32(np.float32(1) / np.float32(B)) / np.float32(D))
    assert a.shape == (B, D) and np.array_equal(a, np.full((B, D), want, np.float32))
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.array_equal(hf.view(np.uint32), hc.view(np.uint32))
    assert_close(hf, 2 * xv.astype(np.float64) / (B * D), "gradient of mean(x*x)", scale=1.0)
    # the gradient of a plain sum: ones, with no reduction evaluated at all
    (ones,) = c.grad([c.sum_all(x)], [x])
    assert ones.op_name == "FilledLike" and np.array_equal(ones.eval({"x": xv}), np.ones((B, D), np.float32))


def test_cross_entropy_gradient_is_built_on_the_logits(G, orc, rng):
    """The gradient of sparse_softmax_cross_entropy is one node over the logits (not over the forward's log-softmax
    output), with the constant of a batch mean handed to its kernel as an argument; a data-dependent upstream gradient
    goes in as an array.  Values against the oracle's two-step form."""
    rows, classes = 37, 11
    lv = (rng.standard_normal((rows, classes)) * 2).astype(np.float32)
    tv = rng.integers(0, classes, (rows, 1)).astype(np.float32)
    wv = rng.standard_normal((rows, 1)).astype(np.float32)
    env = G.VariableEnvironment()
    c = env.context()
    logits, t, w = c.placeholder("l", [rows, classes]), c.placeholder("t", [rows, 1]), c.placeholder("w", [rows, 1])
    loss = c.sparse_softmax_cross_entropy(logits, t)
    (g_mean,) = c.grad([c.reduce_mean(loss, [0], False)], [logits])
    (g_weighted,) = c.grad([c.sum_all(c.mul(loss, w))], [logits])
    assert g_mean.op_name == "SparseSoftmaxCrossEntropyGradLogits" and g_weighted.op_name == "SparseSoftmaxCrossEntropyGradLogits"
    assert g_mean.num_inputs == 4          # logits, labels, and the constant's two extent sources (both the logits)
    assert g_weighted.num_inputs == 3      # logits, labels, the upstream gradient
    say("cross-entropy gradient from the logits")
    a, b, lossv = c.eval([g_mean, g_weighted, loss], {"l": lv, "t": tv, "w": wv})
    _, olsm = orc.sparse_softmax_xent(lv, tv)
    assert_close(a, orc.sparse_softmax_xent_grad(olsm, tv, np.full((rows, 1), np.float32(1) / np.float32(rows), np.float32)), "mean")
    assert_close(b, orc.sparse_softmax_xent_grad(olsm, tv, wv), "weighted")
    assert lossv.shape == (rows, 1)


def test_updates_that_do_not_wait_for_the_device_equal_waiting_ones(G, rng):
    """Optimizer::update returns once its work is enqueued.  Forty steps in a row, each fed from one host buffer
    that is overwritten as soon as update() returns, must leave the variables with exactly the bits of the same
    forty steps run through eval() (which waits and reads the result back) — the graph of step n+1 is built and
    its feeds are copied while the device still runs step n."""
    def train(waiting):
        r = np.random.default_rng(11)
        env = G.VariableEnvironment()
        wid = env.set("w", r.standard_normal((8, 1, 3, 3)).astype(np.float32) * 0.3)
        bid = env.set("b", np.zeros((1, 8, 1, 1), np.float32))
        adam = G.Adam(env, [wid, bid], alpha=0.01)
        buf = np.empty((16, 1, 12, 12), np.float32)
        for step in range(40):
            buf[:] = r.standard_normal(buf.shape).astype(np.float32)
            c = env.context()
            w, b = c.variable(wid), c.variable(bid)
            x = c.placeholder("x", [-1, 1, 12, 12])
            loss = c.sum_all(c.max_pool2d(c.relu(c.conv2d(x, w, 1, 1) + b), 2, 0, 2))
            gw, gb = c.grad([loss], [w, b])
            if waiting:
                out = c.eval([adam.get_update_op([w, b], [gw, gb], c)], {"x": buf})
                assert not isinstance(out[0], G.OpError)
            else:
                adam.update([w, b], [gw, gb], c, {"x": buf})
            buf[:] = np.nan                                     # the device must not see this
        return env.array(wid), env.array(bid)
    w1, b1 = train(waiting=True)
    w2, b2 = train(waiting=False)
    assert np.isfinite(w1).all() and np.array_equal(w1.view(np.uint32), w2.view(np.uint32))
    assert np.array_equal(b1.view(np.uint32), b2.view(np.uint32))


def _small_training(G, seed, steps=25):
    r = np.random.default_rng(seed)
    env = G.VariableEnvironment()
    wid = env.set("w", r.standard_normal((8, 1, 3, 3)).astype(np.float32) * 0.3)
    bid = env.set("b", np.zeros((1, 8, 1, 1), np.float32))
    adam = G.Adam(env, [wid, bid], alpha=0.01)
    for step in range(steps):
        xv = r.standard_normal((16, 1, 12, 12)).astype(np.float32)
        c = env.context()
        w, b = c.variable(wid), c.variable(bid)
        x = c.placeholder("x", [-1, 1, 12, 12])
        loss = c.sum_all(c.max_pool2d(c.relu(c.conv2d(x, w, 1, 1) + b), 2, 0, 2))
        gw, gb = c.grad([loss], [w, b])
        adam.update([w, b], [gw, gb], c, {"x": xv})
    return env.array(wid), env.array(bid)


def test_four_host_threads_train_at_once_each_on_its_own_stream(G):
    """Every host thread that evaluates graphs has a stream, a staging ring and arena lists of its own (the
    reference's graphs live on one thread each, src/graph.rs:17-47).  Four threads train four small models at the
    same time; each must end with exactly the bits of the same training run alone."""
    import threading
    want = {seed: _small_training(G, seed) for seed in range(4)}
    got, errors = {}, []

    def work(seed):
        try:
            got[seed] = _small_training(G, seed)
        except Exception as e:                       # a failure in a thread must fail the test, not vanish
            errors.append((seed, repr(e)[:300]))

    say("four host threads, four trainings through the host layer")
    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for seed in range(4):
        for a, b in zip(got[seed], want[seed]):
            assert np.isfinite(a).all() and np.array_equal(a.view(np.uint32), b.view(np.uint32)), f"thread {seed}"


def test_arrays_handed_from_one_thread_to_another_are_ordered(G, orc):
    """An environment created on one thread, trained on a second and read on the first: each thread's work is ordered
    on its own stream, and an array that another thread's stream used last makes the next user wait for that stream
    (no host synchronisation is needed between the hand-offs beyond joining the thread)."""
    import threading
    r = np.random.default_rng(3)
    env = G.VariableEnvironment()
    wv = r.standard_normal((64, 512)).astype(np.float32)
    wv = (np.sign(wv) * (4.0 + np.abs(wv))).astype(np.float32)   # far from zero: three steps of 0.5 keep the sign
    wid = env.set("w", wv)                      # uploaded on the main thread's stream, not waited for
    adam = G.Adam(env, [wid], alpha=0.5)
    errors = []

    def work():
        try:
            for _ in range(3):
                c = env.context()
                w = c.variable(wid)
                (gw,) = c.grad([c.sum_all(c.mul(w, w))], [w])
                adam.update([w], [gw], c)       # returns once enqueued on the worker's stream
        except Exception as e:
            errors.append(repr(e)[:300])

    say("environment handed between two threads")
    t = threading.Thread(target=work)
    t.start()
    t.join()
    assert not errors, errors
    c = env.context()                           # back on the main thread: reads what the worker's stream wrote
    w = c.variable(wid)
    (sq,) = c.eval([c.mul(w, w)])
    final = env.array(wid)
    p, m, v, t = wv.copy(), np.zeros_like(wv), np.zeros_like(wv), np.ones(1, np.float32)
    for _ in range(3):
        orc.adam(p, (p + p).astype(np.float32), m, v, t, alpha=0.5)
    assert_close(final, p, "w after three steps on another thread")
    assert np.abs(final - wv).min() > 0.1 and np.array_equal(sq, final * final)


def test_batched_adam_updates_keep_the_evaluation_order(G, orc, rng):
    """The AdamOp nodes of one evaluation go out as one launch, but a node that reads a variable after its
    AdamOp ran must see the updated array, exactly as if every update had run at its own node.  The evaluator
    visits the last requested tensor first (src/evaluation.rs:267-272), so in [read, update] the update runs
    before the read and in [update, read] after it."""
    for update_first in (True, False):
        env = G.VariableEnvironment()
        wv = rng.random((6, 5), dtype=np.float32) + 1.0
        bv = rng.random((1, 5), dtype=np.float32) + 1.0
        wid, bid = env.set("w", wv), env.set("b", bv)
        adam = G.Adam(env, [wid, bid], alpha=0.25)
        c = env.context()
        w, b = c.variable(wid), c.variable(bid)
        gw, gb = c.grad([c.sum_all(c.mul(w, w)) + c.sum_all(c.mul(b, b))], [w, b])
        update = adam.get_update_op([w, b], [gw, gb], c)
        read = c.mul(w, w)
        wanted = [read, update] if update_first else [update, read]
        out = c.eval(wanted)
        got = out[0] if update_first else out[1]
        p, m, v, t = wv.copy(), np.zeros_like(wv), np.zeros_like(wv), np.ones(1, np.float32)
        orc.adam(p, (wv + wv).astype(np.float32), m, v, t, alpha=0.25)
        assert_close(env.array(wid), p, "w after the step")
        if update_first:
            assert np.array_equal(got, env.array(wid) ** 2), "the read ran after the update and sees the new array"
        else:
            assert np.array_equal(got, wv * wv), "the read ran before the update and sees the old array"
        pb, mb, vb = bv.copy(), np.zeros_like(bv), np.zeros_like(bv)
        orc.adam(pb, (bv + bv).astype(np.float32), mb, vb, np.ones(1, np.float32), alpha=0.25)
        assert_close(env.array(bid), pb, "b after the step")


def test_updates_queued_before_a_panicking_node_are_still_applied(G, orc, rng):
    """The AdamOp nodes of an evaluation are queued and launched together.  When a later node of the same evaluation
    panics (a placeholder that was fed an array of another shape), the updates queued before it have happened as far
    as the reference is concerned -- each AdamOp runs at its own node, src/evaluation.rs:310-329 -- so the
    evaluation applies them on its way out."""
    env = G.VariableEnvironment()
    wv = rng.random((6, 5), dtype=np.float32) + 1.0
    wid = env.set("w", wv)
    adam = G.Adam(env, [wid], alpha=0.25)
    c = env.context()
    w = c.variable(wid)
    (gw,) = c.grad([c.sum_all(c.mul(w, w))], [w])
    update = adam.get_update_op([w], [gw], c)
    bad = c.relu(c.placeholder("q", [3, 3]))
    say("an evaluation that panics after its update node")
    with pytest.raises(G.Panic):
        c.eval([bad, update], {"q": np.zeros((2, 2), np.float32)})   # the last tensor is visited first
    p, m, v, t = wv.copy(), np.zeros_like(wv), np.zeros_like(wv), np.ones(1, np.float32)
    orc.adam(p, (wv + wv).astype(np.float32), m, v, t, alpha=0.25)
    assert_close(env.array(wid), p, "w after the interrupted evaluation")


# ------------------------------------------------------------------------------- the reference's own gradient tests
def check_theoretical_grads(G, env, c, objective, gradients, var_ids, eps=1e-2, tol=2e-2):
    """src/test_helper.rs:9-140: the analytic gradients of sum_all(objective) w.r.t. shared variables
    against central differences obtained by rewriting the variable in place and re-evaluating the
    same graph.  The reference runs this in f64 with eps 1e-3 / tol 1e-2; in f32 the step is ten
    times larger so that rounding of the objective (about 1e-6 relative) stays below the tolerance."""
    obj = c.sum_all(objective)
    th = c.eval(gradients)
    for vid, g_th in zip(var_ids, th):
        assert not isinstance(g_th, G.OpError), g_th
        base = env.array(vid)
        flat = base.reshape(-1)
        assert g_th.size == flat.size
        for i in range(flat.size):
            vals = []
            for sgn in (+1.0, -1.0):
                pert = flat.copy()
                pert[i] += sgn * eps
                env.write(vid, pert.reshape(base.shape))
                vals.append(float(c.eval([obj])[0]))
            env.write(vid, base)
            g_num = (vals[0] - vals[1]) / (2 * eps)
            assert abs(g_num - float(g_th.reshape(-1)[i])) <= tol * max(1.0, abs(g_num)), (
                f"gradient check: numerical={g_num}, theoretical={g_th.reshape(-1)[i]} at element {i}")


def ref_env(G, rng, shapes):
    env = G.VariableEnvironment()
    ids = [env.set(f"v{i}", rng.standard_normal(s).astype(np.float32)) for i, s in enumerate(shapes)]
    return env, ids


def test_ref_conv2d_transpose(G, rng):                      # tests/test_tensor_ops_grad.rs:1358
    env, (xi, wi) = ref_env(G, rng, [(3, 2, 2, 2), (2, 3, 2, 2)])
    c = env.context()
    x, w = c.variable(xi), c.variable(wi)
    y = c.conv2d_transpose(x, w, 0, 1)
    check_theoretical_grads(G, env, c, y, c.grad([y], [w]), [wi])


def test_ref_conv2d_transpose_filter_grad(G, rng):          # :1374 (second order; the answer is zero)
    env, (xi, wi) = ref_env(G, rng, [(2, 2, 2, 2), (2, 3, 2, 2)])
    c = env.context()
    x, w = c.variable(xi), c.variable(wi)
    y = c.conv2d_transpose(x, w, 0, 1)
    g = c.grad([y], [w])[0]
    check_theoretical_grads(G, env, c, g, c.grad([g], [w]), [wi])


def test_ref_conv2d_filter_grad(G, rng):                    # :1399 (second order; the answer is zero)
    env, (xi, wi) = ref_env(G, rng, [(2, 3, 5, 5), (2, 3, 2, 2)])
    c = env.context()
    x, w = c.variable(xi), c.variable(wi)
    y = c.conv2d(x, w, 0, 1)
    g = c.grad([y], [w])[0]
    check_theoretical_grads(G, env, c, g, c.grad([g], [w]), [wi])


def test_ref_conv2d_grad(G, rng):                           # :1423 grad_with_default, then w.r.t. gy
    env, (xi, wi) = ref_env(G, rng, [(2, 3, 5, 5), (2, 3, 2, 2)])
    # The reference feeds ones of shape [2,2,2,2] although y is [2,2,4,4]; its input gradient then
    # has the extent rebuilt from gy (3x3).  Here the gradient takes x's extent, so gy has y's shape.
    gyi = env.set("gy", np.ones((2, 2, 4, 4), np.float32))
    c = env.context()
    x, w, gy = c.variable(xi), c.variable(wi), c.variable(gyi)
    y = c.conv2d(x, w, 0, 1)
    g = c.grad_with_default([y], [x], [gy])[0]
    check_theoretical_grads(G, env, c, g, [c.grad([g], [gy])[0]], [gyi])


def test_ref_conv2d_xw_grad(G, rng):                        # :1449 d(filter grad)/dx
    env, (xi, wi) = ref_env(G, rng, [(2, 3, 5, 5), (2, 3, 2, 2)])
    c = env.context()
    x, w = c.variable(xi), c.variable(wi)
    y = c.conv2d(x, w, 0, 1)
    g = c.grad([y], [w])[0]
    check_theoretical_grads(G, env, c, g, c.grad([g], [x]), [xi])


def test_ref_conv2d(G, rng):                                # :1473 pad 1, stride 2
    env, (xi, wi) = ref_env(G, rng, [(2, 3, 5, 5), (2, 3, 3, 3)])
    c = env.context()
    x, w = c.variable(xi), c.variable(wi)
    y = c.conv2d(x, w, 1, 2)
    check_theoretical_grads(G, env, c, y, c.grad([y], [x, w]), [xi, wi])


def test_ref_max_pool2d(G):                                 # :1496
    env = G.VariableEnvironment()
    xi = env.set("x", np.linspace(0.0, 1.0, 9, dtype=np.float32))
    c = env.context()
    x = c.variable(xi)
    y = c.max_pool2d(c.reshape(x, [1, 1, 3, 3]), 2, 0, 1)
    check_theoretical_grads(G, env, c, y, c.grad([y], [x]), [xi])


def test_ref_max_pool2d_grad(G):                            # :1508 runs MaxPool2DGradGrad
    env = G.VariableEnvironment()
    xi = env.set("x", np.linspace(0.0, 1.0, 36, dtype=np.float32))
    gyi = env.set("gy", np.linspace(0.0, 1.0, 16, dtype=np.float32).reshape(2, 2, 2, 2))
    c = env.context()
    x, gy = c.variable(xi), c.variable(gyi)
    y = c.max_pool2d(c.reshape(x, [2, 2, 3, 3]), 2, 0, 1)
    g = c.grad_with_default([y], [x], [gy])[0]
    check_theoretical_grads(G, env, c, g, [c.grad([g], [gy])[0]], [gyi])


def test_ref_matmul_and_batch_matmul(G, rng):               # :457, :479
    env, (ai, bi) = ref_env(G, rng, [(4, 2), (2, 3)])
    c = env.context()
    a, b = c.variable(ai), c.variable(bi)
    z = c.matmul(a, b)
    check_theoretical_grads(G, env, c, z, c.grad([z], [a, b]), [ai, bi])
    env, (ai, bi) = ref_env(G, rng, [(2, 4, 2), (2, 2, 3)])
    c = env.context()
    a, b = c.variable(ai), c.variable(bi)
    z = c.batch_matmul(a, b)
    check_theoretical_grads(G, env, c, z, c.grad([z], [a, b]), [ai, bi])


def test_ref_reduce_and_wx_plus_b(G, rng):                  # :523, :627-:690
    env, (xi,) = ref_env(G, rng, [(3, 2, 3)])
    for keep in (False, True):
        for op in ("reduce_mean", "reduce_sum"):
            c = env.context()
            x = c.variable(xi)
            z = getattr(c, op)(x, [1], keep)
            check_theoretical_grads(G, env, c, z, c.grad([z], [x]), [xi])
    env, (xi, wi, bi) = ref_env(G, rng, [(2, 3), (3, 4), (1, 4)])
    c = env.context()
    x, w, b = c.variable(xi), c.variable(wi), c.variable(bi)
    z = c.matmul(x, w) + b
    check_theoretical_grads(G, env, c, z, c.grad([z], [b]), [bi])


# ------------------------------------------------------------------------------- saved environments
def test_ref_save_and_load(G, rng, tmp_path):                # src/variable.rs:811-841
    path = str(tmp_path / "model.json")
    env = G.VariableEnvironment()
    a = rng.standard_normal((2, 3)).astype(np.float32)
    b = rng.standard_normal((2, 3)).astype(np.float32)
    ida, idb = env.set("a", a), env.set("b", b)
    env.save(path)
    loaded = G.VariableEnvironment.load(path)
    assert len(loaded) == len(env) == 2
    for vid, want in ((ida, a), (idb, b)):
        # the reference asserts 1e-6; shortest-round-trip digits give the same bits back
        assert loaded.array(vid).tobytes() == want.tobytes()
    assert loaded.find("a") == ida and loaded.find("b") == idb and loaded.find("c") is None


def test_ref_save_and_init(G, rng, tmp_path):                # src/variable.rs:843-866
    path = str(tmp_path / "model.json")
    env = G.VariableEnvironment()
    a = env.set("a", rng.standard_normal((2, 3)).astype(np.float32))
    b = env.set("b", rng.standard_normal((2, 3)).astype(np.float32))
    before = [env.array(a), env.array(b)]
    for _ in range(10):
        c = env.context()
        c.variable(a), c.variable(b)
        env.save(path)            # saving from inside a run, over the previous file
    env.initialize(path)
    assert [env.array(a).tobytes(), env.array(b).tobytes()] == [x.tobytes() for x in before]


def test_training_resumes_identically_from_a_saved_environment(G, rng, tmp_path):
    # parameters in the default namespace, Adam's m/v/t in the optimizer's namespace, every shape
    # rank (0-d t, 4-d filter); a run that is saved, reloaded and continued must match one that
    # was never interrupted, bit for bit
    path = str(tmp_path / "train.json")
    x = rng.standard_normal((4, 2, 8, 8)).astype(np.float32)

    def make():
        r = np.random.default_rng(3)
        env = G.VariableEnvironment()
        wid = env.set("w", (0.3 * r.standard_normal((3, 2, 3, 3))).astype(np.float32))
        bid = env.set("b", np.zeros((1, 3, 1, 1), np.float32), namespace="bias")
        return env, wid, bid

    def step(env, adam, wid, bid):
        c = env.context()
        w, b = c.variable(wid), c.variable(bid)
        y = c.relu(c.add(c.conv2d(c.placeholder("x", [-1, 2, 8, 8]), w, 1, 1), b))
        loss = c.sum_all(c.mul(y, y))
        gw, gb = c.grad([loss], [w, b])
        adam.update([w, b], [gw, gb], c, feeds={"x": x})

    env1, wid, bid = make()
    adam1 = G.Adam(env1, [wid, bid], alpha=0.05)
    for _ in range(4):
        step(env1, adam1, wid, bid)

    env2, _, _ = make()
    adam2 = G.Adam(env2, [wid, bid], alpha=0.05)
    for _ in range(2):
        step(env2, adam2, wid, bid)
    env2.save(path)
    text = open(path).read()
    assert text.startswith('{"array_list":[{"v":1,"dim":[3,2,3,3],"data":[') and '"bias\\u0001b":1' in text
    env3 = G.VariableEnvironment.load(path)
    assert len(env3) == len(env2) and env3.find("b", namespace="bias") == bid
    for vid in range(len(env2)):
        assert env3.array(vid).tobytes() == env2.array(vid).tobytes(), f"loaded variable {vid}"
    # Adam::new always registers fresh m, v, t (src/optimizers/adam.rs:84-101), so a run is continued
    # with the optimizer it already has, after `initialize` put the saved arrays back in place
    for _ in range(3):
        step(env2, adam2, wid, bid)     # wander off ...
    env2.initialize(path)               # ... and come back to the saved state
    for _ in range(2):
        step(env2, adam2, wid, bid)
    for vid in range(len(env1)):
        assert env2.array(vid).tobytes() == env1.array(vid).tobytes(), f"variable {vid}"


def test_a_name_registered_twice_is_bound_to_the_newer_array(G):   # src/variable.rs:347-358
    env = G.VariableEnvironment()
    first = env.set("w", np.zeros((2,), np.float32))
    second = env.set("w", np.ones((3,), np.float32))
    assert (first, second) == (0, 1) and env.find("w") == second and len(env) == 2
    assert env.array(first).shape == (2,) and env.array(second).shape == (3,)


@pytest.mark.parametrize("shape,bshape", [((4, 3, 6, 6), (1, 3, 1, 1)), ((5, 7), (5, 1)), ((3, 4, 5), (1, 1, 1)),
                                          ((3, 4, 5), (1, 4, 1))])
def test_add_broadcast_and_the_reduced_gradient(G, rng, shape, bshape):
    # AddOp with ndarray broadcasting of a unit-extent operand and MaybeReduceSum
    # (binary_ops.rs:39-105, 147-166): d sum(w * (x + b)) / db = w summed over the broadcast axes
    x = rng.standard_normal(shape).astype(np.float32)
    b = rng.standard_normal(bshape).astype(np.float32)
    w = rng.standard_normal(shape).astype(np.float32)
    env = G.VariableEnvironment()
    c = env.context()
    xt, bt, wt = (c.variable(env.set(n, a)) for n, a in (("x", x), ("b", b), ("w", w)))
    y = c.add(xt, bt)
    gx, gb = c.grad([c.mul(y, wt)], [xt, bt])
    yv, gxv, gbv = c.eval([y, gx, gb])
    assert np.array_equal(yv, x + b)
    assert np.array_equal(gxv, w)
    axes = tuple(i for i, (s, t) in enumerate(zip(shape, bshape)) if t == 1 and s > 1)
    want = w.astype(np.float64).sum(axis=axes, keepdims=True)
    assert gbv.shape == tuple(bshape)
    assert_close(gbv, want, "bias gradient", scale=np.abs(w).astype(np.float64).sum(axis=axes, keepdims=True))


# ------------------------------------------------------------------------------- column-free convolution in the graph
@pytest.mark.parametrize("B,Cin,Cout,H,k,pad", [(64, 32, 64, 32, 3, 1), (24, 64, 128, 36, 3, 1), (32, 32, 32, 28, 5, 2),
                                               (64, 32, 64, 36, 3, 0), (56, 32, 32, 32, 3, 2)])   # and without / with more than "same" padding
def test_conv2d_column_free_through_the_graph(G, orc, rng, B, Cin, Cout, H, k, pad):
    # channel counts that are multiples of 32, "same" stride-1 convolution: Conv2D keeps a zero-bordered
    # input instead of the columns and all three operators run column-free; values against the oracle
    xv = rng.standard_normal((B, Cin, H, H)).astype(np.float32)
    wv = glorot(rng, (Cout, Cin, k, k))
    env = G.VariableEnvironment()
    c = env.context()
    x, w = c.placeholder("x", list(xv.shape)), c.placeholder("w", list(wv.shape))
    y = c.conv2d(x, w, pad, 1)
    gx, gw = c.grad([c.sum_all(c.mul(y, y))], [x, w])
    second = c.nth_tensor(y, 1)
    say(f"column-free conv through the graph B={B} C={Cin} K={Cout} H={H} k={k}")
    yv, gxv, gwv, kept = c.eval([y, gx, gw, second], {"x": xv, "w": wv})
    assert kept.ndim == 1, "Conv2D is expected to keep the bordered input, not the columns, at this shape"
    oy, ocols = orc.conv2d_fwd(xv, wv, pad, 1, 1)
    assert_close(yv, oy, "y", scale=1.0)
    gyv = (2 * yv).astype(np.float32)
    assert_close(gwv, orc.conv2d_filter_grad(ocols, gyv, wv.shape), "gw", scale=np.abs(gwv).max())
    assert_close(gxv, orc.conv2d_transpose(gyv, wv, pad, 1, 1, out_hw=(H, H)), "gx", scale=np.abs(gxv).max())


@pytest.mark.parametrize("B,Cin,Cout,H,k,pad,d", [(64, 32, 64, 32, 3, 2, 2), (40, 64, 32, 30, 3, 3, 3)])
def test_dilated_conv2d_column_free_through_the_graph(G, orc, rng, B, Cin, Cout, H, k, pad, d):
    # a dilated "same" stride-1 convolution large enough for Conv2D to go column-free: the kept second output is
    # the bordered input (rank 1) and the three operators read their taps `d` apart; `columns=True` keeps the
    # reference's columns, and both agree with the oracle
    xv = rng.standard_normal((B, Cin, H, H)).astype(np.float32)
    wv = glorot(rng, (Cout, Cin, k, k))
    oy, ocols = orc.conv2d_fwd(xv, wv, pad, 1, d)
    gyv = (2 * oy).astype(np.float32)
    ogw = orc.conv2d_filter_grad(ocols, gyv, wv.shape)
    ogx = orc.conv2d_transpose(gyv, wv, pad, 1, d, out_hw=(H, H))
    for columns in (False, True):
        env = G.VariableEnvironment()
        c = env.context()
        x, w = c.placeholder("x", list(xv.shape)), c.placeholder("w", list(wv.shape))
        y = c.dilated_conv2d(x, w, pad, 1, d, columns=columns)
        gx, gw = c.grad([c.sum_all(c.mul(y, y))], [x, w])
        say(f"dilated conv through the graph B={B} C={Cin} K={Cout} H={H} d={d} columns={columns}")
        yv, gxv, gwv, kept = c.eval([y, gx, gw, c.nth_tensor(y, 1)], {"x": xv, "w": wv})
        assert (kept.ndim == 1) == (not columns)
        assert_close(yv, oy, "y", scale=1.0)
        assert_close(gwv, ogw, "gw", scale=np.abs(ogw).max())
        assert_close(gxv, ogx, "gx", scale=np.abs(ogx).max())


@pytest.mark.parametrize("H", [32, 33])
def test_conv2d_stride2_column_free_through_the_graph_and_the_column_switch(G, orc, rng, H):
    # stride 2 at a size where Conv2D goes column-free: the kept second output is the phase-split input
    # (rank 1), the filter gradient reads x's extents from its extra input (28 outputs fit both 55 and 56
    # input rows), and `columns=True` makes the same operator keep the reference's columns instead
    B, Cin, Cout, k, pad = 240, 32, 64, 3, 1   # 17.7 M column elements: above the size from which Conv2D goes column-free
    xv = rng.standard_normal((B, Cin, H, H)).astype(np.float32)
    wv = glorot(rng, (Cout, Cin, k, k))
    oy, ocols = orc.conv2d_fwd(xv, wv, pad, 2, 1)
    gyv = (2 * oy).astype(np.float32)
    ogw = orc.conv2d_filter_grad(ocols, gyv, wv.shape)
    ogx = orc.conv2d_transpose(gyv, wv, pad, 2, 1, out_hw=(H, H))
    for columns in (False, True):
        env = G.VariableEnvironment()
        c = env.context()
        x, w = c.placeholder("x", list(xv.shape)), c.placeholder("w", list(wv.shape))
        y = c.conv2d(x, w, pad, 2, columns=columns)
        gx, gw = c.grad([c.sum_all(c.mul(y, y))], [x, w])
        say(f"stride-2 conv through the graph H={H} columns={columns}")
        yv, gxv, gwv, kept = c.eval([y, gx, gw, c.nth_tensor(y, 1)], {"x": xv, "w": wv})
        assert (kept.ndim == 1) == (not columns)
        if columns:
            assert np.array_equal(kept.reshape(ocols.shape), ocols)
        assert_close(yv, oy, "y", scale=1.0)
        assert_close(gwv, ogw, "gw", scale=np.abs(ogw).max())
        assert_close(gxv, ogx, "gx", scale=np.abs(ogx).max())


@pytest.mark.parametrize("stride,H", [(1, 32), (2, 64)])
def test_both_gradients_of_a_column_free_conv_share_the_bordered_gradient(G, rng, stride, H):
    # the filter gradient and the input gradient read the same zero-bordered copy of gy: evaluated together, the second
    # of them finds the copy the first one made; evaluated apart, each makes its own -- same bits either way.  A filter
    # that Adam has rewritten in between is not served from a copy made for its old values.
    B, Cin, Cout, k, pad = 64, 32, 64, 3, 1
    xv = rng.standard_normal((B, Cin, H, H)).astype(np.float32)
    env = G.VariableEnvironment()
    wid = env.set("w", glorot(rng, (Cout, Cin, k, k)))
    adam = G.Adam(env, [wid], alpha=1e-2)

    def graph():
        c = env.context()
        x, w = c.placeholder("x", list(xv.shape)), c.variable(wid)
        y = c.conv2d(x, w, pad, stride)
        gx, gw = c.grad([c.sum_all(c.mul(y, y))], [x, w])
        return c, w, y, gx, gw

    for step in range(2):
        say(f"shared bordered gradient stride={stride} step={step}")
        c, w, y, gx, gw = graph()
        before = G.reused_copies()
        gxv, gwv, kept = c.eval([gx, gw, c.nth_tensor(y, 1)], {"x": xv})
        assert kept.ndim == 1, "the convolution is expected to run column-free at this size"
        assert G.reused_copies() == before + 1
        c1, _, _, gx1, _ = graph()
        c2, _, _, _, gw2 = graph()
        before = G.reused_copies()
        assert np.array_equal(c1.eval([gx1], {"x": xv})[0], gxv)
        assert np.array_equal(c2.eval([gw2], {"x": xv})[0], gwv)
        assert G.reused_copies() == before
        # one Adam step on the filter, then everything again with the new values
        c3, w3, _, _, gw3 = graph()
        adam.update([w3], [gw3], c3, {"x": xv})


@pytest.mark.parametrize("B", [4, 64])
def test_a_convolution_over_a_variable_equals_one_over_a_fed_array(G, rng, B):
    # the gradients of conv -> 2x2 pooling take their output extents from the forward inputs through ExtentsOf nodes
    # (an array with a shape and no elements); over a variable that must neither copy the variable nor change a bit
    # (B = 4: over columns; B = 64: column-free)
    C, K, H = 32, 32, 32
    xv = rng.standard_normal((B, C, H, H)).astype(np.float32)
    wv = glorot(rng, (K, C, 3, 3))
    got = []
    for as_variable in (False, True):
        env = G.VariableEnvironment()
        wid = env.set("w", wv)
        c = env.context()
        x = c.variable(env.set("x", xv)) if as_variable else c.placeholder("x", list(xv.shape))
        w = c.variable(wid)
        y = c.max_pool2d(c.conv2d(x, w, 1, 1), 2, 0, 2)
        grads = c.grad([c.sum_all(c.mul(y, y))], [x, w])
        say(f"convolution over a {'variable' if as_variable else 'fed array'}, B={B}")
        got.append(c.eval([y] + grads, None if as_variable else {"x": xv}))
        assert np.array_equal(env.array(wid), wv)
    for a, b in zip(*got):
        assert np.array_equal(a, b)


def test_a_conv_relu_pool_conv_chain_has_the_same_bits_with_and_without_the_evaluators_shortcuts(G, rng):
    # conv -> ReLU(+bias) -> 2x2 pooling -> conv, both convolutions column-free, loss = sum of squares: the evaluator runs
    # each ReLU inside its pooling's launch and each convolution's two gradients off one bordered copy of gy; with the
    # shortcuts switched off every node runs on its own.  Values, gradients and an Adam step: the same bits.
    B, C1, C2, H = 32, 32, 64, 64
    xv = rng.standard_normal((B, C1, H, H)).astype(np.float32)
    w1v, w2v = glorot(rng, (C2, C1, 3, 3)), glorot(rng, (C2, C2, 3, 3))
    bv = (0.1 * rng.standard_normal((1, C2, 1, 1))).astype(np.float32)
    results = []
    for on in (True, False):
        G.set_shortcuts(on)
        try:
            env = G.VariableEnvironment()
            ids = [env.set("w1", w1v), env.set("w2", w2v), env.set("b", bv)]
            adam = G.Adam(env, ids, alpha=1e-2)
            c = env.context()
            x = c.placeholder("x", list(xv.shape))
            w1, w2, b = (c.variable(i) for i in ids)
            z = c.max_pool2d(c.relu(c.conv2d(x, w1, 1, 1) + b), 2, 0, 2)
            y = c.conv2d(z, w2, 1, 1)
            loss = c.sum_all(c.mul(y, y))
            grads = c.grad([loss], [x, w1, w2, b])
            say(f"conv-relu-pool-conv chain, shortcuts {'on' if on else 'off'}")
            reused = G.reused_copies()
            vals = c.eval([y, z] + grads, {"x": xv})
            assert (c.fused_pairs, G.reused_copies() - reused) == ((1, 2) if on else (0, 0))
            c2 = env.context()
            x = c2.placeholder("x", list(xv.shape))
            w1, w2, b = (c2.variable(i) for i in ids)
            y = c2.conv2d(c2.max_pool2d(c2.relu(c2.conv2d(x, w1, 1, 1) + b), 2, 0, 2), w2, 1, 1)
            adam.update([w1, w2, b], c2.grad([c2.sum_all(c2.mul(y, y))], [w1, w2, b]), c2, {"x": xv})
            vals += [env.array(i) for i in ids]
            results.append(vals)
        finally:
            G.set_shortcuts(True)
    for a, b_ in zip(*results):
        assert np.array_equal(a, b_)


def test_conv2d_column_free_second_order(G, orc, rng):
    # the gradient of the filter gradient: w.r.t. x (Conv2DTranspose of the incoming gradient) and
    # w.r.t. gy (Conv2DWithCols, here over the bordered input)
    B, Cin, Cout, H = 64, 32, 32, 32   # 18.9 M column elements: above the size from which Conv2D goes column-free
    xv = rng.standard_normal((B, Cin, H, H)).astype(np.float32)
    wv = glorot(rng, (Cout, Cin, 3, 3))
    rv = rng.standard_normal(wv.shape).astype(np.float32)
    env = G.VariableEnvironment()
    c = env.context()
    x, w, r = (c.placeholder(n, list(a.shape)) for n, a in (("x", xv), ("w", wv), ("r", rv)))
    y = c.conv2d(x, w, 1, 1)
    gys = c.mul(y, y)
    (gw,) = c.grad([c.sum_all(gys)], [w])          # gw = filter_grad(x, gy = 2y)
    (ggx,) = c.grad([c.sum_all(c.mul(gw, r))], [x])
    say("column-free second order")
    gwv, ggxv, kept = c.eval([gw, ggx, c.nth_tensor(y, 1)], {"x": xv, "w": wv, "r": rv})
    assert kept.ndim == 1, "Conv2D is expected to keep the bordered input at this shape"
    # f(x) = <filter_grad(x, 2 conv(x, w)), r>; with gy = 2 conv(x, w):
    # df/dx = conv_transpose(gy, r) + conv_transpose(2 conv(x, r), w)
    oy, ocols = orc.conv2d_fwd(xv, wv, 1, 1, 1)
    gyv = (2 * oy).astype(np.float32)
    assert_close(gwv, orc.conv2d_filter_grad(ocols, gyv, wv.shape), "gw", scale=np.abs(gwv).max())
    oyr, _ = orc.conv2d_fwd(xv, rv, 1, 1, 1)
    want = orc.conv2d_transpose(gyv, rv, 1, 1, 1, out_hw=(H, H)).astype(np.float64) + \
        orc.conv2d_transpose((2 * oyr).astype(np.float32), wv, 1, 1, 1, out_hw=(H, H)).astype(np.float64)
    assert_close(ggxv, want, "ggx", scale=np.abs(want).max())


def test_many_steps_with_changing_batch_sizes_do_not_grow_memory(G, rng):
    # the evaluator's arena and the staging ring are reused from step to step: after a warm-up that has seen every
    # batch size, hundreds of further training steps of the small CNN (graph rebuilt and fed every step, Adam
    # update, batch size changing from step to step) leave the device's used memory and the process's peak host
    # memory where they were
    import resource

    import torch
    env = G.VariableEnvironment()
    params = {"w1": glorot(rng, (32, 1, 3, 3)), "w2": glorot(rng, (64, 32, 3, 3)),
              "w3": rng.uniform(-0.04, 0.04, (3136, 10)).astype(np.float32),
              "b1": np.zeros((1, 32, 28, 28), np.float32), "b2": np.zeros((1, 64, 14, 14), np.float32),
              "b3": np.zeros((1, 10), np.float32)}
    ids = {k: env.set(k, a) for k, a in params.items()}
    names = list(params)
    adam = G.Adam(env, [ids[k] for k in names], alpha=1e-3)
    sizes = [128, 64, 100, 128, 32]

    def step(bs):
        c = env.context()
        v = {k: c.variable(ids[k]) for k in names}
        x, t = c.placeholder("x", [-1, 1, 28, 28]), c.placeholder("y", [-1, 1])
        z = c.max_pool2d(c.relu(c.conv2d(x, v["w1"], 1, 1) + v["b1"]), 2, 0, 2)
        z = c.max_pool2d(c.relu(c.conv2d(z, v["w2"], 1, 1) + v["b2"]), 2, 0, 2)
        logits = c.matmul(c.reshape(z, [-1, 3136]), v["w3"]) + v["b3"]
        loss = c.reduce_mean(c.sparse_softmax_cross_entropy(logits, t), [0], False)
        grads = c.grad([loss], [v[k] for k in names])
        adam.update([v[k] for k in names], grads, c,
                    {"x": rng.random((bs, 1, 28, 28), dtype=np.float32),
                     "y": rng.integers(0, 10, (bs, 1)).astype(np.float32)})

    def used():
        G.synchronize()
        free, total = torch.cuda.mem_get_info()
        return total - free, resource.getrusage(resource.RUSAGE_SELF).ru_maxrss

    say("memory over many steps: warm-up")
    for i in range(40):
        step(sizes[i % 5])
    dev0, host0 = used()
    say("memory over many steps: 400 steps")
    for i in range(400):
        step(sizes[i % 5])
    dev1, host1 = used()
    assert dev1 - dev0 <= 8 << 20, (dev0, dev1)          # bytes; other tests' torch tensors may be freed meanwhile
    assert host1 - host0 <= 16 << 10, (host0, host1)     # KiB


def test_conv2d_and_gradients_through_the_graph_random_geometries_exact(G, orc):
    # Conv2D with any stride, dilation and padding, channel counts on both sides of what the column-free paths take
    # and batches on both sides of the operator's size switch: y, gx and gw through the graph (whichever path the
    # operator picks) against the CPU restatement, small integers, bit for bit
    r = np.random.default_rng(20241127)
    for _ in range(40):
        s_, k, d = int(r.choice([1, 1, 2])), int(r.choice([2, 3, 3, 5])), int(r.choice([1, 1, 2]))
        reach = d * (k - 1)
        p = int(r.integers(0, reach + 1))
        B, C, Kc = int(r.choice([1, 3, 8, 40, 150])), int(r.choice([3, 32, 64, 96])), int(r.choice([8, 32, 64, 160]))
        H, W = int(r.integers(max(reach + 1, 6), 50)), int(r.integers(max(reach + 1, 6), 50))
        while B * max(C, Kc) * H * W > 8e6:
            B = max(B // 2, 1)
        geo = (B, C, Kc, H, W, k, p, s_, d)
        x = r.integers(-3, 4, (B, C, H, W)).astype(np.float32)
        w = r.integers(-2, 3, (Kc, C, k, k)).astype(np.float32)
        oy, ocols = orc.conv2d_fwd(x, w, p, s_, d)
        m = r.integers(-2, 3, oy.shape).astype(np.float32)
        say(f"conv2d through the graph, random geometry {geo}")
        env = G.VariableEnvironment()
        wid = env.set("w", w)
        c = env.context()
        xt, wt = c.placeholder("x", [-1, C, H, W]), c.variable(wid)
        mt = c.placeholder("m", [-1] + list(oy.shape[1:]))
        y = c.dilated_conv2d(xt, wt, p, s_, d)
        gx, gw = c.grad([c.sum_all(c.mul(y, mt))], [xt, wt])
        vy, vgx, vgw = c.eval([y, gx, gw], {"x": x, "m": m})
        assert np.array_equal(vy, oy), geo
        assert np.array_equal(vgx, orc.conv2d_transpose(m, w, p, s_, d, out_hw=(H, W))), geo
        assert np.array_equal(vgw, orc.conv2d_filter_grad(ocols, m, w.shape)), geo
