"""Pins the CPU oracle (oracle/ag_oracle.c) before it is trusted as the checker.

Three kinds of evidence, none of which re-types the oracle's own formula:
  * the known-answer vectors the reference's tests hold (tests/golden/reference_vectors.json),
  * independent library routines on the CPU (torch.nn.functional conv / pool in f64, numpy matmul),
  * what the mathematics fixes: brute-force index definitions, the im2col/col2im adjoint identity,
    closed forms for reductions and for the first Adam step.
"""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F


def _allclose(a, b, rtol=1e-4, atol=1e-5):
    np.testing.assert_allclose(np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64),
                               rtol=rtol, atol=atol)


# ----------------------------------------------------------------------------- im2col / col2im
def test_im2col_reference_vector(orc, golden):
    g = golden["im2col_batch"]
    img = np.array(g["x_per_image"], dtype=np.float32).reshape(g["xch"], g["xh"], g["xw"])
    x = np.stack([img] * g["batch"])
    cols = orc.im2col(x, g["kh"], g["kw"], g["pad"], g["pad"], g["stride"], g["stride"],
                      g["dilation"], g["dilation"])
    assert cols.reshape(-1).tolist() == [float(v) for v in g["expected"]]


def _im2col_bruteforce(x, kh, kw, p, s, d):
    B, C, H, W = x.shape
    OH = (H + 2 * p - (d * (kh - 1) + 1)) // s + 1
    OW = (W + 2 * p - (d * (kw - 1) + 1)) // s + 1
    out = np.zeros((B, C, kh, kw, OH, OW), dtype=x.dtype)
    for b, c, ky, kx, oy, ox in itertools.product(range(B), range(C), range(kh), range(kw),
                                                  range(OH), range(OW)):
        iy, ix = oy * s - p + ky * d, ox * s - p + kx * d
        if 0 <= iy < H and 0 <= ix < W:
            out[b, c, ky, kx, oy, ox] = x[b, c, iy, ix]
    return out.reshape(B, C * kh * kw, OH * OW)


GEOMS = [  # H, W, kh, kw, pad, stride, dil
    (5, 5, 3, 3, 1, 1, 1), (5, 5, 3, 3, 1, 2, 1), (7, 6, 3, 2, 0, 1, 1), (8, 8, 3, 3, 2, 1, 2),
    (9, 7, 2, 3, 1, 3, 1), (6, 6, 4, 4, 1, 2, 1), (4, 4, 1, 1, 0, 1, 1), (10, 10, 3, 3, 3, 2, 3),
]


@pytest.mark.parametrize("geom", GEOMS)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_im2col_matches_index_definition(orc, rng, geom, dtype):
    H, W, kh, kw, p, s, d = geom
    x = rng.standard_normal((2, 3, H, W)).astype(dtype)
    got = orc.im2col(x, kh, kw, p, p, s, s, d, d)
    assert np.array_equal(got, _im2col_bruteforce(x, kh, kw, p, s, d))


def test_im2col_matches_torch_unfold(orc, rng):
    x = rng.standard_normal((2, 4, 9, 8))
    got = orc.im2col(x, 3, 3, 1, 1, 2, 2, 1, 1)
    want = F.unfold(torch.from_numpy(x), kernel_size=3, dilation=1, padding=1, stride=2).numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("geom", GEOMS)
def test_col2im_is_adjoint_of_im2col(orc, rng, geom):
    H, W, kh, kw, p, s, d = geom
    x = rng.standard_normal((2, 3, H, W))
    cols = orc.im2col(x, kh, kw, p, p, s, s, d, d)
    c = rng.standard_normal(cols.shape)
    OH, OW = orc.conv_out_size(H, kh, p, s, d), orc.conv_out_size(W, kw, p, s, d)
    back = orc.col2im(c, 3, H, W, kh, kw, p, p, s, s, d, d, OH, OW)
    _allclose(np.vdot(cols, c), np.vdot(x, back), rtol=1e-12, atol=1e-12)


def test_col2im_matches_torch_fold(orc, rng):
    c = rng.standard_normal((2, 4 * 9, 5 * 4))
    got = orc.col2im(c, 4, 9, 8, 3, 3, 1, 1, 2, 2, 1, 1, 5, 4)
    want = F.fold(torch.from_numpy(c), output_size=(9, 8), kernel_size=3, padding=1, stride=2).numpy()
    _allclose(got, want, rtol=1e-12, atol=1e-12)


def test_col2im_f32_sums_in_kernel_position_order(orc):
    """f32 additions at one pixel happen in (ky, kx) ascending order: pick values whose f32 sum
    depends on the order (1e8 + 1 - 1e8)."""
    kh = kw = 3
    cols = np.zeros((1, 9, 9), dtype=np.float32)  # C=1, 3x3 image, pad 1 -> 3x3 outputs
    # centre pixel (1,1) receives cols[ky,kx] at output (1-ky+1, 1-kx+1) = (2-ky, 2-kx)
    vals = [1e8, 1.0, -1e8, 1.0, 0.5, 0.25, 3.0, -2.0, 7.0]
    for k, v in enumerate(vals):
        ky, kx = divmod(k, 3)
        cols[0, k, (2 - ky) * 3 + (2 - kx)] = v
    got = orc.col2im(cols, 1, 3, 3, kh, kw, 1, 1, 1, 1, 1, 1, 3, 3)[0, 0, 1, 1]
    acc = np.float32(0)
    for v in vals:
        acc = np.float32(acc + np.float32(v))
    assert got == acc
    assert got != np.float32(sum(sorted(vals)))  # a different order gives a different f32


# ----------------------------------------------------------------------------- conv ops
def test_deconv_reference_vector(orc, golden):
    g = golden["deconv"]
    w = np.ones(g["w_shape"], dtype=np.float32)
    gy = np.ones(g["g_shape"], dtype=np.float32)
    out = orc.conv2d_transpose(gy, w, g["pad"], g["stride"], 1)
    assert list(out.shape) == g["expected_shape"]
    for b in range(out.shape[0]):
        for c in range(out.shape[1]):
            assert out[b, c].reshape(-1).tolist() == [float(v) for v in g["expected_plane"]]


CONV_CASES = [  # B, C, K, H, W, k, pad, stride, dil
    (2, 3, 4, 5, 5, 3, 1, 2, 1),   # geometry of tests/test_tensor_ops_grad.rs:1473-1493
    (2, 2, 3, 6, 7, 3, 1, 1, 1),
    (1, 4, 2, 9, 9, 3, 2, 1, 2),
    (3, 1, 5, 8, 8, 2, 0, 2, 1),
    (2, 3, 3, 7, 7, 4, 1, 3, 1),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_forward_and_grads_match_torch_f64(orc, rng, case):
    B, C, K, H, W, k, p, s, d = case
    x = rng.standard_normal((B, C, H, W))
    w = rng.standard_normal((K, C, k, k))
    xt = torch.from_numpy(x).requires_grad_()
    wt = torch.from_numpy(w).requires_grad_()
    yt = F.conv2d(xt, wt, padding=p, stride=s, dilation=d)
    gy = rng.standard_normal(tuple(yt.shape))
    yt.backward(torch.from_numpy(gy))

    y, cols = orc.conv2d_fwd(x, w, p, s, d)
    _allclose(y, yt.detach().numpy(), rtol=1e-11, atol=1e-11)
    gw = orc.conv2d_filter_grad(cols, gy, w.shape)
    _allclose(gw, wt.grad.numpy(), rtol=1e-11, atol=1e-11)
    gx = orc.conv2d_transpose(gy, w, p, s, d, out_hw=(H, W))
    _allclose(gx, xt.grad.numpy(), rtol=1e-11, atol=1e-11)
    # Conv2DWithCols is the GEMM half of the forward
    _allclose(orc.conv2d_with_cols(cols, w, y.shape[2], y.shape[3]), y, rtol=1e-12, atol=1e-12)

    # f32 instance agrees with the f64 truth to the stated tolerance
    y32, cols32 = orc.conv2d_fwd(x.astype(np.float32), w.astype(np.float32), p, s, d)
    _allclose(y32, y, rtol=1e-4, atol=1e-5)
    assert np.array_equal(cols32, cols.astype(np.float32))


def test_conv2d_transpose_reconstructed_size_is_a_crop(orc, rng):
    """When (H + 2p - k_eff) % s != 0 the reference's reconstructed input extent is smaller than
    the true one and its result equals the top-left crop of the true gradient."""
    B, C, K, H, W, k, p, s, d = 2, 2, 3, 8, 8, 3, 1, 2, 1  # OH = 4 -> reconstructed 7
    gy = rng.standard_normal((B, K, 4, 4))
    w = rng.standard_normal((K, C, k, k))
    small = orc.conv2d_transpose(gy, w, p, s, d)
    assert small.shape == (B, C, 7, 7)
    full = orc.conv2d_transpose(gy, w, p, s, d, out_hw=(H, W))
    _allclose(small, full[:, :, :7, :7], rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("case", [(2, 3, 2, 4, 4, 2, 0, 1, 1), (2, 4, 3, 5, 5, 4, 1, 2, 1),
                                  (1, 2, 2, 3, 3, 3, 1, 1, 1)])
def test_conv2d_transpose_and_its_filter_grad_match_torch(orc, rng, case):
    B, ych, xch, yh, yw, k, p, s, d = case
    x = rng.standard_normal((B, ych, yh, yw))          # input of the transposed conv
    w = rng.standard_normal((ych, xch, k, k))
    xt = torch.from_numpy(x).requires_grad_()
    wt = torch.from_numpy(w).requires_grad_()
    ot = F.conv_transpose2d(xt, wt, padding=p, stride=s, dilation=d)
    go = rng.standard_normal(tuple(ot.shape))
    ot.backward(torch.from_numpy(go))

    out = orc.conv2d_transpose(x, w, p, s, d)
    assert out.shape == tuple(ot.shape)
    _allclose(out, ot.detach().numpy(), rtol=1e-11, atol=1e-11)
    gw = orc.conv2d_transpose_filter_grad(x, go, w.shape, p, s, d)
    _allclose(gw, wt.grad.numpy(), rtol=1e-11, atol=1e-11)
    # gradient w.r.t. the transposed conv's input is a plain Conv2D of go with w
    gx, _ = orc.conv2d_fwd(go, w, p, s, d)
    _allclose(gx, xt.grad.numpy(), rtol=1e-11, atol=1e-11)


# ----------------------------------------------------------------------------- GEMM family
def _mk(entry, key):
    if key + "_ones" in entry:
        return np.ones(entry[key + "_ones"], dtype=np.float32)
    return np.array(entry[key], dtype=np.float32)


def test_matmul_reference_vectors(orc, golden):
    for e in golden["matmul"]:
        c = orc.matmul(_mk(e, "a"), _mk(e, "b"), e["ta"], e["tb"])
        assert c.reshape(-1).tolist() == [float(v) for v in e["expected"]], e["source"]


def test_batch_matmul_reference_vectors(orc, golden):
    for e in golden["batch_matmul"]:
        c = orc.batch_matmul(_mk(e, "a"), _mk(e, "b"), e["ta"], e["tb"])
        if "expected_fill" in e:
            assert list(c.shape) == e["expected_shape"]
            assert np.all(c == e["expected_fill"])
        else:
            assert np.array_equal(c, np.array(e["expected"], dtype=np.float32)), e["source"]


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_matches_numpy_with_leading_dims_and_beta(orc, rng, ta, tb):
    m, n, k = 7, 9, 11
    lda, ldb, ldc = (m if ta else k) + 3, (k if tb else n) + 2, n + 4
    a = rng.standard_normal(((k if ta else m), lda))
    b = rng.standard_normal(((n if tb else k), ldb))
    c0 = rng.standard_normal((m, ldc))
    A = a[:, :m].T if ta else a[:, :k]
    Bm = b[:, :k].T if tb else b[:, :n]
    want = c0.copy()
    want[:, :n] = 0.5 * A @ Bm - 1.5 * c0[:, :n]
    for naive in (True, False):
        c = c0.copy()
        orc.gemm(ta, tb, m, n, k, 0.5, a, lda, b, ldb, -1.5, c, ldc, naive=naive)
        _allclose(c, want, rtol=1e-12, atol=1e-12)


def test_gemm_blocked_path_and_openblas_agree_with_numpy(orc, rng):
    a = rng.standard_normal((300, 500)).astype(np.float32)
    b = rng.standard_normal((500, 480)).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64)
    orc.unload_blas()
    _allclose(orc.matmul(a, b), want, rtol=1e-4, atol=1e-4)     # 72 M MACs -> blocked loops
    if orc.load_openblas():
        assert "openblas" in orc.blas_name().lower()
        _allclose(orc.matmul(a, b), want, rtol=1e-4, atol=1e-4)
        _allclose(orc.matmul(a.T.copy(), b.T.copy(), True, True), want, rtol=1e-4, atol=1e-4)
        orc.unload_blas()


# ----------------------------------------------------------------------------- max pooling
def test_max_pool_reference_vector(orc, golden):
    g = golden["max_pool"]
    x = np.array(g["x"], dtype=np.float64).reshape(g["batch"], g["ch"], g["xh"], g["xw"])
    y, am, il = orc.maxpool2d_fwd(x, g["size"], g["pad"], g["stride"])
    assert y.reshape(-1).tolist() == [float(v) for v in g["expected_output"]]
    assert am.reshape(-1).tolist() == [float(v) for v in g["expected_argmax"]]
    assert il.reshape(-1).tolist() == g["expected_argmax"]


def _pool_bruteforce(x, size, stride):
    B, C, H, W = x.shape
    OH, OW = (H - size) // stride + 1, (W - size) // stride + 1
    y = np.empty((B, C, OH, OW), dtype=x.dtype)
    idx = np.empty((B, C, OH, OW), dtype=np.int64)
    flat = x.reshape(-1)
    for b, c, oy, ox in itertools.product(range(B), range(C), range(OH), range(OW)):
        best, best_i = -np.finfo(x.dtype).max, 0
        for h in range(oy * stride, oy * stride + size):
            for w in range(ox * stride, ox * stride + size):
                i = ((b * C + c) * H + h) * W + w
                if flat[i] > best:
                    best, best_i = flat[i], i
        y[b, c, oy, ox], idx[b, c, oy, ox] = best, best_i
    return y, idx


@pytest.mark.parametrize("H,W,size,stride", [(6, 6, 2, 2), (7, 9, 3, 2), (8, 8, 3, 1), (5, 7, 2, 3)])
def test_max_pool_matches_bruteforce_and_torch(orc, rng, H, W, size, stride):
    x = rng.standard_normal((2, 3, H, W)).astype(np.float32)
    y, am, il = orc.maxpool2d_fwd(x, size, 0, stride)
    wy, widx = _pool_bruteforce(x, size, stride)
    assert np.array_equal(y, wy)
    assert np.array_equal(am, widx.astype(np.float32))
    ty, tidx = F.max_pool2d(torch.from_numpy(x), size, stride, return_indices=True)
    assert np.array_equal(y, ty.numpy())
    assert np.array_equal(il, tidx.numpy().astype(np.int32))   # torch indices are plane-local


def test_max_pool_ties_nan_and_floor(orc):
    x = np.zeros((1, 2, 4, 4), dtype=np.float32)            # all ties: first element of the window
    x[0, 1] = np.nan                                         # NaN never beats the start value
    y, am, il = orc.maxpool2d_fwd(x, 2, 0, 2)
    assert am[0, 0].reshape(-1).tolist() == [0.0, 2.0, 8.0, 10.0]
    assert np.all(y[0, 1] == -np.finfo(np.float32).max) and np.all(am[0, 1] == 0.0)
    assert np.all(il[0, 1] == -1)
    with pytest.raises(ValueError):
        orc.maxpool2d_fwd(x, 2, 1, 2)


def test_max_pool_float_encoded_index_rounds_above_2_pow_24(orc):
    """The index is stored by value in the element type: above 2**24 an f32 cannot hold it."""
    B, C, H, W = 1, 1, 4100, 4100                            # 16.81 M elements > 2**24
    x = np.zeros((B, C, H, W), dtype=np.float32)
    x[0, 0, 4099, 4097] = 1.0                                # flat index 16 809 997 (odd)
    y, am, il = orc.maxpool2d_fwd(x, 2, 0, 2)
    flat = 4099 * W + 4097
    assert il[0, 0, -1, -2] == flat
    assert am[0, 0, -1, -2] == np.float32(flat) and int(am[0, 0, -1, -2]) != flat


@pytest.mark.parametrize("H,W,size,stride", [(6, 6, 2, 2), (7, 9, 3, 2), (8, 8, 3, 1)])
def test_max_pool_backward_matches_torch_and_gradgrad_is_gather(orc, rng, H, W, size, stride):
    x = rng.standard_normal((2, 3, H, W))
    xt = torch.from_numpy(x).requires_grad_()
    yt = F.max_pool2d(xt, size, stride)
    gy = rng.standard_normal(tuple(yt.shape))
    yt.backward(torch.from_numpy(gy))
    y, am, il = orc.maxpool2d_fwd(x, size, 0, stride)
    gx, skipped = orc.maxpool2d_bwd(gy, am, x.shape)
    assert skipped == 0
    _allclose(gx, xt.grad.numpy(), rtol=1e-12, atol=1e-12)
    assert np.array_equal(orc.maxpool2d_bwd_local(gy, il, x.shape), gx)
    ggx = rng.standard_normal(x.shape)
    ggy = orc.maxpool2d_gradgrad(ggx, am, y.shape)
    assert np.array_equal(ggy, ggx.reshape(-1)[am.astype(np.int64)])


def test_max_pool_backward_with_reference_reconstructed_size_drops_out_of_range(orc, rng):
    """3x3 stride-2 pooling of a 6x6 plane: the reference sizes gx as 2*(2-1)+3 = 5x5 = 25 elements
    per plane while indices address the 6x6 tensor; the oracle reports such writes instead of
    performing them."""
    x = rng.standard_normal((1, 1, 6, 6))
    x[0, 0, 4, 4] = 10.0                                     # flat index 28 >= 25
    y, am, il = orc.maxpool2d_fwd(x, 3, 0, 2)
    n = orc.pool_grad_in_size(2, 3, 0, 2)
    assert n == 5
    _, skipped = orc.maxpool2d_bwd(np.ones_like(y), am, (1, 1, n, n))
    assert skipped >= 1


# ----------------------------------------------------------------------------- reductions
def test_reduce_mean_reference_value(orc, golden):
    g = golden["reduce_mean"]
    out = orc.reduce_mean(np.array(g["x"], dtype=np.float32), g["axes"], g["keep_dims"])
    assert out.shape == () and float(out) == g["expected"]


def test_sum_all_closed_form_and_order(orc):
    n = 4099
    x = np.arange(1, n + 1, dtype=np.float32)
    assert orc.sum_all(x) == np.float32(n * (n + 1) // 2)     # exact in f32 (< 2**24)
    assert orc.sum_all(np.zeros(0, dtype=np.float32)) == 0
    # eight-lane order: lanes 0 and 4 are combined before anything else
    y = np.zeros(16, dtype=np.float32)
    y[0], y[4], y[1] = 1e8, -1e8, 1.0
    assert orc.sum_all(y) == np.float32(1.0)                  # (1e8 + -1e8) first, then + 1
    z = np.zeros(16, dtype=np.float32)
    z[0], z[1], z[4] = 1e8, 1.0, -1e8
    assert orc.sum_all(z) == orc.sum_all(y)


@pytest.mark.parametrize("axes", [[0], [1], [2], [3], [0, 2], [1, 3], [0, 1, 2, 3], [-1], [3, 0]])
@pytest.mark.parametrize("keep", [False, True])
def test_reduce_sum_and_mean_match_numpy(orc, rng, axes, keep):
    x = rng.standard_normal((3, 4, 5, 6))
    ax = tuple(a % 4 for a in axes)
    _allclose(orc.reduce_sum(x, axes, keep), x.sum(axis=ax, keepdims=keep), rtol=1e-12, atol=1e-12)
    _allclose(orc.reduce_mean(x, axes, keep), x.mean(axis=ax, keepdims=keep), rtol=1e-12, atol=1e-12)
    assert orc.reduce_sum(x, axes, keep).shape == x.sum(axis=ax, keepdims=keep).shape


def test_reduce_sum_f32_is_sequential_along_the_axis(orc):
    x = np.array([[1e8, 1.0, -1e8, 1.0]], dtype=np.float32)
    acc = np.float32(0)
    for v in x[0]:
        acc = np.float32(acc + v)
    assert orc.reduce_sum(x, [1])[0] == acc == np.float32(1.0)


def test_reduce_mean_multiplies_by_f32_reciprocal(orc):
    x = np.full((3, 1), 7.0, dtype=np.float32)
    want = np.float32(np.float32(21.0) * (np.float32(1.0) / np.float32(3.0)))
    assert orc.reduce_mean(x, [0])[0] == want


def test_broadcast_grad(orc, rng):
    gy = rng.standard_normal((3, 1, 5, 1))
    got = orc.broadcast_grad(gy, (3, 4, 5, 6), [1, 3])
    assert np.array_equal(got, np.broadcast_to(gy, (3, 4, 5, 6)))
    s = np.array(2.5)
    assert np.all(orc.broadcast_grad(s, (2, 3), [0, 1]) == 2.5)


# ----------------------------------------------------------------------------- Adam
def test_adam_first_step_closed_form(orc, rng):
    """From m = v = 0 and t = 1 the bias-corrected moments are g and g*g, so the step is
    -alpha * g / (|g| + eps), independent of b1 and b2."""
    g = rng.standard_normal(1000)
    p0 = rng.standard_normal(1000)
    p, m, v, t = p0.copy(), np.zeros(1000), np.zeros(1000), np.array([1.0])
    orc.adam(p, g, m, v, t, alpha=1e-3, eps=1e-8, b1=0.9, b2=0.999)
    _allclose(p, p0 - 1e-3 * g / (np.abs(g) + 1e-8), rtol=1e-9, atol=1e-12)
    _allclose(m, 0.1 * g, rtol=1e-12, atol=0)
    _allclose(v, 0.001 * g * g, rtol=1e-9, atol=0)
    assert t[0] == 2.0


def test_adam_multi_step_recurrence(orc, rng):
    n, steps = 257, 5
    a, e, b1, b2 = 2e-3, 1e-8, 0.8, 0.95
    p = rng.standard_normal(n)
    m, v, t = np.zeros(n), np.zeros(n), np.array([1.0])
    rp, rm, rv = p.copy(), m.copy(), v.copy()
    p32, m32, v32, t32 = (p.astype(np.float32), m.astype(np.float32), v.astype(np.float32),
                          np.array([1.0], dtype=np.float32))
    for k in range(1, steps + 1):
        g = rng.standard_normal(n)
        orc.adam(p, g, m, v, t, a, e, b1, b2)
        orc.adam(p32, g.astype(np.float32), m32, v32, t32, a, e, b1, b2)
        rm = b1 * rm + (1 - b1) * g
        rv = b2 * rv + (1 - b2) * g * g
        rp = rp - a * (rm / (1 - b1 ** k)) / (np.sqrt(rv / (1 - b2 ** k)) + e)
    _allclose(p, rp, rtol=1e-10, atol=1e-12)
    _allclose(p32, rp, rtol=1e-4, atol=1e-5)
    assert t[0] == steps + 1 and t32[0] == steps + 1


# ----------------------------------------------------------------------------- glue
def test_relu_add_bias_add_n(orc, rng):
    x = rng.standard_normal((7, 5)).astype(np.float32)
    gy = rng.standard_normal((7, 5)).astype(np.float32)
    assert np.array_equal(orc.relu(x), np.maximum(x, 0))
    assert np.array_equal(orc.relu_grad(x, gy), np.where(x > 0, gy, np.float32(0)))
    b = rng.standard_normal(5).astype(np.float32)
    assert np.array_equal(orc.add_bias(x, b), x + b)
    xs = [rng.standard_normal(33).astype(np.float32) for _ in range(4)]
    assert np.array_equal(orc.add_n(xs), ((xs[0] + xs[1]) + xs[2]) + xs[3])


def test_sparse_softmax_xent_matches_torch(orc, rng):
    logits = rng.standard_normal((16, 10)) * 3
    labels = rng.integers(0, 10, size=(16, 1)).astype(np.float64)
    lt = torch.from_numpy(logits).requires_grad_()
    loss_t = F.cross_entropy(lt, torch.from_numpy(labels.reshape(-1)).long(), reduction="none")
    gy = rng.standard_normal((16, 1))
    loss_t.backward(torch.from_numpy(gy.reshape(-1)))
    loss, lsm = orc.sparse_softmax_xent(logits, labels)
    assert loss.shape == (16, 1)
    _allclose(loss.reshape(-1), loss_t.detach().numpy(), rtol=1e-12, atol=1e-12)
    _allclose(lsm, F.log_softmax(lt, dim=1).detach().numpy(), rtol=1e-12, atol=1e-12)
    _allclose(orc.sparse_softmax_xent_grad(lsm, labels, gy), lt.grad.numpy(), rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("pad,stride,dil,k", [(1, 1, 1, 3), (1, 2, 1, 3), (2, 1, 2, 3), (1, 2, 1, 4), (0, 1, 1, 2)])
def test_direct_definitions_used_by_the_full_size_gpu_tests(orc, rng, pad, stride, dil, k):
    """tests/direct_conv.py (sampled f64 truth of the B = 256 GPU tests) against the oracle: every
    output element of a small case."""
    from direct_conv import direct_gw, direct_gx, direct_y
    B, C, Kf, H = 3, 5, 4, 11
    x = rng.standard_normal((B, C, H, H))
    w = rng.standard_normal((Kf, C, k, k))
    y, cols = orc.conv2d_fwd(x, w, pad, stride, dil)
    OH = y.shape[2]
    gy = rng.standard_normal(y.shape)
    idx = np.array([(b, f, oy, ox) for b in range(B) for f in range(Kf) for oy in range(OH) for ox in range(OH)])
    assert np.allclose(direct_y(x, w, idx, pad, stride, dil), y.reshape(-1), rtol=1e-12, atol=1e-12)
    gx = orc.conv2d_transpose(gy, w, pad, stride, dil, out_hw=(H, H))
    idx = np.array([(b, c, iy, ix) for b in range(B) for c in range(C) for iy in range(H) for ix in range(H)])
    assert np.allclose(direct_gx(gy, w, idx, pad, stride, dil), gx.reshape(-1), rtol=1e-12, atol=1e-12)
    gw = orc.conv2d_filter_grad(cols, gy, w.shape)
    ch = np.array([1, 3])
    assert np.allclose(direct_gw(x, gy, ch, k, k, pad, stride, dil), gw[:, ch], rtol=1e-12, atol=1e-12)
