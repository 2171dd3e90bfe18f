"""Parity at the benchmark configurations' FULL sizes (through the C ABI, one GPU):

  config 3   4096^3 MatMul in the NN / NT / TN layouts and 64 x 512^3 BatchMatMul with both operand
             gradients, against numpy's f64 product of the same arrays, plus integer-valued inputs
             (exact in f32) for equality;
  config 4   B = 256, 64 -> 128 channels, 56 x 56, 3 x 3, stride 1 AND stride 2: y, gw and gx against
             the direct definition of the convolution evaluated in f64 on a random sample of output
             elements (gw: all filters and taps of sampled input channels, each the full sum over the
             256 images), plus integer-valued inputs for equality; 3 x 3 stride-2 max pooling forward
             and backward on the full [256,128,56,56] against the oracle, bit for bit;
  config 5   32 images: dilation-2 convolution and the 4 x 4 stride-2 transposed convolution,
             forward and both gradients, against the f64 oracle.

The schedules that only exist at these sizes (a dozen rounds of the persistent grid plus the
narrow-tile tail, the 256-way split fold) are thereby checked against something other than
themselves.  Bars: tests/bars.py.
"""
import numpy as np
import pytest
import torch

from bars import assert_contraction, say
from direct_conv import direct_gw, direct_gx, direct_y

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    import __graft_entry__ as entry
    entry.load_package()
    from rust_autograd_amd import kernels
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return kernels


@pytest.fixture(scope="module", autouse=True)
def reference_blas(orc):
    path = orc.load_openblas()
    say("oracle BLAS:", path or "built-in blocked GEMM")
    yield path
    orc.unload_blas()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.detach().cpu().numpy()


# ------------------------------------------------------------------------------------- config 3
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False)])
def test_config3_matmul_4096(K, ta, tb):
    n = 4096
    rng = np.random.default_rng(4096 + 2 * ta + tb)
    a = rng.standard_normal((n, n)).astype(np.float32)
    b = rng.standard_normal((n, n)).astype(np.float32)
    say("matmul 4096^3", ta, tb)
    got = host(K.matmul(dev(a), dev(b), ta, tb))
    A = (a.T if ta else a).astype(np.float64)
    Bm = (b.T if tb else b).astype(np.float64)
    ref32 = (a.T if ta else a) @ (b.T if tb else b)            # numpy's f32 product (OpenBLAS sgemm)
    assert_contraction(got, A @ Bm, np.abs(A) @ np.abs(Bm), f"matmul 4096^3 ta={ta} tb={tb}", ref32=ref32)
    del A, Bm
    ai = rng.integers(-3, 4, (n, n)).astype(np.float32)
    bi = rng.integers(-3, 4, (n, n)).astype(np.float32)
    exact = (ai.T if ta else ai) @ (bi.T if tb else bi)         # every partial sum < 2^24: exact in any order
    assert np.array_equal(host(K.matmul(dev(ai), dev(bi), ta, tb)), exact)


def test_config3_batch_matmul_64x512_with_both_gradients(K):
    rng = np.random.default_rng(64512)
    a = rng.standard_normal((64, 512, 512)).astype(np.float32)
    b = rng.standard_normal((64, 512, 512)).astype(np.float32)
    gy = np.ones((64, 512, 512), np.float32)     # grad() of a sum: dot_ops.rs:697-717 with gy = ones
    a64, b64, g64 = (v.astype(np.float64) for v in (a, b, gy))
    say("batch_matmul 64x512^3")
    z = host(K.batch_matmul(dev(a), dev(b)))
    assert_contraction(z, a64 @ b64, np.abs(a64) @ np.abs(b64), "batch_matmul z", ref32=a @ b)
    ga = host(K.batch_matmul(dev(gy), dev(b), False, True))      # gy . b^T
    assert_contraction(ga, g64 @ b64.transpose(0, 2, 1), g64 @ np.abs(b64).transpose(0, 2, 1), "batch_matmul ga",
                       ref32=gy @ b.transpose(0, 2, 1))
    gb = host(K.batch_matmul(dev(a), dev(gy), True, False))      # a^T . gy
    assert_contraction(gb, a64.transpose(0, 2, 1) @ g64, np.abs(a64).transpose(0, 2, 1) @ g64, "batch_matmul gb",
                       ref32=a.transpose(0, 2, 1) @ gy)
    ai = rng.integers(-3, 4, a.shape).astype(np.float32)
    bi = rng.integers(-3, 4, b.shape).astype(np.float32)
    assert np.array_equal(host(K.batch_matmul(dev(ai), dev(bi))), ai @ bi)
    assert np.array_equal(host(K.batch_matmul(dev(ai), dev(bi), True, False)), ai.transpose(0, 2, 1) @ bi)
    assert np.array_equal(host(K.batch_matmul(dev(ai), dev(bi), False, True)), ai @ bi.transpose(0, 2, 1))


# ------------------------------------------------------------------------------------- config 4
def _conv_paths(K, x, w, gy, pad, stride, dil):
    """(y, gw, gx) of the operator path the host layer takes for this geometry, and of the column path."""
    H, W = x.shape[2:]
    out = {}
    y, cols = K.conv2d(x, w, pad, stride, dil)
    gw = K.conv2d_filter_grad(cols, gy, tuple(w.shape))
    del cols
    gx = K.conv2d_transpose(gy, w, pad, stride, dil, out_hw=(H, W), return_cols=True)[0]
    out["columns"] = (y, gw, gx)
    res = K.conv2d_nocols(x, w, pad, stride, dil)
    staged = K.conv_input_grad_staged(gy, w, pad, (H, W), stride, dil)
    if res is not None and staged is not None:
        gw2 = K.conv2d_filter_grad_nocols(res[1], staged[1], tuple(x.shape), tuple(w.shape), pad, stride, dil)
        out["column-free"] = (res[0], gw2, staged[0])
        del res, staged
        # the input gradient through the operator entry point, which picks the column-free route itself
        out["column-free, operator entry"] = (out["column-free"][0], gw2, K.conv2d_transpose(gy, w, pad, stride, dil, out_hw=(H, W)))
    return out


@pytest.mark.parametrize("stride", [1, 2])
def test_config4_conv_b256_against_direct_definition(K, orc, stride):
    B, C, Kf, H, k, pad = 256, 64, 128, 56, 3, 1
    OH = (H + 2 * pad - k) // stride + 1
    rng = np.random.default_rng(256 + stride)
    sc = np.sqrt(6.0 / Kf)
    x = rng.standard_normal((B, C, H, H)).astype(np.float32)
    w = rng.uniform(-sc, sc, (Kf, C, k, k)).astype(np.float32)
    gy = rng.standard_normal((B, Kf, OH, OH)).astype(np.float32)
    assert stride == 1 or K.conv2d_nocols(dev(x[:2]), dev(w), pad, stride) is not None, "stride 2 is expected to be column-free too"
    n = 8192
    yi = np.stack([rng.integers(0, B, n), rng.integers(0, Kf, n), rng.integers(0, OH, n), rng.integers(0, OH, n)], 1)
    xi = np.stack([rng.integers(0, B, n), rng.integers(0, C, n), rng.integers(0, H, n), rng.integers(0, H, n)], 1)
    # make sure image borders and the last image are in the sample
    yi[:64, 2] = 0; yi[64:128, 3] = OH - 1; yi[128:192, 0] = B - 1
    xi[:64, 2] = H - 1; xi[64:128, 3] = 0; xi[128:192, 0] = B - 1
    chans = np.sort(rng.choice(C, 8, replace=False))
    say("config 4 B=256 stride", stride, "host truth")
    y_t, y_a = direct_y(x, w, yi, pad, stride, 1), direct_y(np.abs(x), np.abs(w), yi, pad, stride, 1)
    gx_t, gx_a = direct_gx(gy, w, xi, pad, stride, 1), direct_gx(np.abs(gy), np.abs(w), xi, pad, stride, 1)
    gw_t, gw_a = direct_gw(x, gy, chans, k, k, pad, stride, 1), direct_gw(np.abs(x), np.abs(gy), chans, k, k, pad, stride, 1)
    # the reference's own arithmetic on the whole batch: the f32 oracle (im2col, SGEMM through OpenBLAS where it is
    # loaded, image-sequential filter gradient, col2im), sampled at the same elements -- bars 2 and 3 at the shape
    # the headline metric is quoted on
    say("config 4 B=256 stride", stride, "f32 oracle on the whole batch")
    o_y, o_cols = orc.conv2d_fwd(x, w, pad, stride, 1, threads=16)
    o_gw = orc.conv2d_filter_grad(o_cols, gy, w.shape)
    del o_cols
    o_gx = orc.conv2d_transpose(gy, w, pad, stride, 1, out_hw=(H, H), threads=16)
    y_32, gx_32, gw_32 = o_y[tuple(yi.T)], o_gx[tuple(xi.T)], o_gw[:, chans]
    del o_y, o_gx
    for name, (y, gw, gx) in _conv_paths(K, dev(x), dev(w), dev(gy), pad, stride, 1).items():
        say("config 4 B=256 stride", stride, name)
        yv, gwv, gxv = host(y), host(gw), host(gx)
        assert_contraction(yv[tuple(yi.T)], y_t, y_a, f"stride {stride} {name} y", ref32=y_32)
        assert_contraction(gxv[tuple(xi.T)], gx_t, gx_a, f"stride {stride} {name} gx", ref32=gx_32)
        assert_contraction(gwv[:, chans], gw_t, gw_a, f"stride {stride} {name} gw", ref32=gw_32)
    # integer-valued data: every partial sum is an integer below 2^24, so f32 is exact in any order
    x = rng.integers(-3, 4, x.shape).astype(np.float32)
    w = rng.integers(-2, 3, w.shape).astype(np.float32)
    gy = rng.integers(-2, 3, gy.shape).astype(np.float32)
    y_t, gx_t, gw_t = direct_y(x, w, yi, pad, stride, 1), direct_gx(gy, w, xi, pad, stride, 1), direct_gw(x, gy, chans, k, k, pad, stride, 1)
    for name, (y, gw, gx) in _conv_paths(K, dev(x), dev(w), dev(gy), pad, stride, 1).items():
        say("config 4 B=256 stride", stride, name, "integers")
        assert np.array_equal(host(y)[tuple(yi.T)], y_t), f"{name} y"
        assert np.array_equal(host(gx)[tuple(xi.T)], gx_t), f"{name} gx"
        assert np.array_equal(host(gw)[:, chans], gw_t), f"{name} gw"


def test_config4_maxpool_full_tensor_bit_exact(K, orc):
    B, C, H = 256, 128, 56
    rng = np.random.default_rng(27)
    x = rng.standard_normal((B, C, H, H)).astype(np.float32)
    x[3, 5, 10:14, 10:14] = 1.5          # ties inside windows: the first maximum in row-major order wins
    say("max_pool2d 3x3 s2 on [256,128,56,56]")
    y, am, il = K.max_pool2d(dev(x), 3, 0, 2)
    oy, oam, oil = orc.maxpool2d_fwd(x, 3, 0, 2)
    assert np.array_equal(host(y), oy)
    assert np.array_equal(host(am).view(np.uint32), oam.view(np.uint32)), "f32-encoded argmax (rounded above 2^24)"
    assert np.array_equal(host(il), orc.maxpool2d_taps(oil, H, 3, 2))
    gy = rng.standard_normal(oy.shape).astype(np.float32)
    gx = host(K.max_pool2d_grad(dev(gy), am, il, x.shape, 3, 0, 2))
    assert np.array_equal(gx.view(np.uint32), orc.maxpool2d_bwd_local(gy, oil, x.shape).view(np.uint32))


# ------------------------------------------------------------------------------------- config 5
def test_config5_dilated_conv_32_images(K, orc):
    B, C, Kf, H, k, pad, dil = 32, 256, 256, 14, 3, 2, 2
    rng = np.random.default_rng(55)
    x = rng.standard_normal((B, C, H, H)).astype(np.float32)
    w = rng.uniform(-0.1, 0.1, (Kf, C, k, k)).astype(np.float32)
    gy = rng.standard_normal((B, Kf, H, H)).astype(np.float32)
    x64, w64, g64 = (v.astype(np.float64) for v in (x, w, gy))
    say("config 5 dilated, 32 images")
    y64, cols64 = orc.conv2d_fwd(x64, w64, pad, 1, dil)
    ya, colsa = orc.conv2d_fwd(np.abs(x64), np.abs(w64), pad, 1, dil)
    y32, cols32 = orc.conv2d_fwd(x, w, pad, 1, dil)
    y, cols = K.conv2d(dev(x), dev(w), pad, 1, dil)
    assert np.array_equal(host(cols), cols32)
    assert_contraction(host(y), y64, ya, "dilated y", ref32=y32)
    gw = host(K.conv2d_filter_grad(cols, dev(gy), w.shape))
    assert_contraction(gw, orc.conv2d_filter_grad(cols64, g64, w.shape), orc.conv2d_filter_grad(colsa, np.abs(g64), w.shape),
                       "dilated gw", ref32=orc.conv2d_filter_grad(cols32, gy, w.shape))
    gx = host(K.conv2d_transpose(dev(gy), dev(w), pad, 1, dil, out_hw=(H, H)))
    assert_contraction(gx, orc.conv2d_transpose(g64, w64, pad, 1, dil, out_hw=(H, H)),
                       orc.conv2d_transpose(np.abs(g64), np.abs(w64), pad, 1, dil, out_hw=(H, H)), "dilated gx",
                       ref32=orc.conv2d_transpose(gy, w, pad, 1, dil, out_hw=(H, H)))


def test_config5_transposed_conv_32_images(K, orc):
    B, ych, xch, h, k, pad, stride = 32, 128, 64, 14, 4, 1, 2
    rng = np.random.default_rng(56)
    x = rng.standard_normal((B, ych, h, h)).astype(np.float32)
    w = rng.uniform(-0.1, 0.1, (ych, xch, k, k)).astype(np.float32)
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    say("config 5 transposed conv, 32 images")
    y = K.conv2d_transpose(dev(x), dev(w), pad, stride)                     # reference-reconstructed 28 x 28
    y64 = orc.conv2d_transpose(x64, w64, pad, stride, 1)
    assert y64.shape == (B, xch, 28, 28) == tuple(y.shape)
    assert_contraction(host(y), y64, orc.conv2d_transpose(np.abs(x64), np.abs(w64), pad, stride, 1), "deconv y",
                       ref32=orc.conv2d_transpose(x, w, pad, stride, 1))
    gy = rng.standard_normal(y64.shape).astype(np.float32)
    g64 = gy.astype(np.float64)
    # gradient w.r.t. the input is a convolution of gy with w (conv2d_transpose.rs:274-300)
    gx, _ = K.conv2d(dev(gy), dev(w), pad, stride, 1)
    gx64, _ = orc.conv2d_fwd(g64, w64, pad, stride, 1)
    assert_contraction(host(gx), gx64, orc.conv2d_fwd(np.abs(g64), np.abs(w64), pad, stride, 1)[0], "deconv gx",
                       ref32=orc.conv2d_fwd(gy, w, pad, stride, 1)[0])
    gw = host(K.conv2d_transpose_filter_grad(dev(x), dev(gy), w.shape, pad, stride))
    assert_contraction(gw, orc.conv2d_transpose_filter_grad(x64, g64, w.shape, pad, stride, 1),
                       orc.conv2d_transpose_filter_grad(np.abs(x64), np.abs(g64), w.shape, pad, stride, 1), "deconv gw",
                       ref32=orc.conv2d_transpose_filter_grad(x, gy, w.shape, pad, stride, 1))


@pytest.mark.parametrize("stride,B", [(1, 1200), (2, 4800)])
def test_conv_batch_whose_columns_exceed_2_pow_31_elements(K, stride, B):
    # 1200 images of the headline shape (4800 at stride 2): 2.17e9 column elements (8.7 GB), past what a 32-bit
    # element index reaches.  Small integers, generated on the device: the column path and the column-free path,
    # which share no indexing code, must agree bit for bit on y, gw and gx; the magnitudes say the sums are not
    # trivially zero.
    C, Kf, H, k, p = 64, 128, 56, 3, 1
    assert B * C * k * k * (H // stride) ** 2 > 2**31
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    x = torch.randint(-3, 4, (B, C, H, H), device="cuda", generator=gen).float()
    w = torch.randint(-2, 3, (Kf, C, k, k), device="cuda", generator=gen).float()
    say("conv2d with 2.17e9 column elements: column-free forward")
    res = K.conv2d_nocols(x, w, p, stride, 1)
    assert res is not None
    say("conv2d with 2.17e9 column elements: column forward")
    y, cols = K.conv2d(x, w, p, stride, 1)
    assert torch.equal(y, res[0]) and float(y.abs().max()) > 50
    gy = torch.randint(-2, 3, tuple(y.shape), device="cuda", generator=gen).float()
    del y
    say("conv2d with 2.17e9 column elements: filter gradients")
    staged = K.conv_input_grad_staged(gy, w, p, (H, H), stride, 1)
    gw = K.conv2d_filter_grad_nocols(res[1], staged[1], tuple(x.shape), tuple(w.shape), p, stride, 1)
    assert torch.equal(gw, K.conv2d_filter_grad(cols, gy, tuple(w.shape))) and float(gw.abs().max()) > 1000
    del cols, res
    say("conv2d with 2.17e9 column elements: input gradients")
    gx_cols, gcols = K.conv2d_transpose(gy, w, p, stride, 1, out_hw=(H, H), return_cols=True)
    del gcols
    assert torch.equal(staged[0], gx_cols)
    del staged, gx_cols, gy, x
    torch.cuda.empty_cache()


def test_max_pool_over_more_than_2_pow_31_elements(K):
    # [1500, 128, 112, 112] = 2.4e9 elements, 2 x 2 windows that do not overlap (every input element receives at most
    # one gradient, so no summation order is involved): values and backward bit for bit against torch's own pooling
    # with its int64 indices, which shares nothing with the kernels here
    import torch.nn.functional as F
    B, C, H, W = 1500, 128, 112, 112
    assert B * C * H * W > 2**31
    gen = torch.Generator(device="cuda")
    gen.manual_seed(2)
    x = torch.randn(B, C, H, W, device="cuda", generator=gen)
    say("max_pool over 2.4e9 elements: forward")
    y, am, taps = K.max_pool2d(x, 2, 0, 2)
    ty, tidx = F.max_pool2d(x, 2, 2, return_indices=True)
    assert torch.equal(y, ty)
    del ty
    gy = torch.randn(tuple(y.shape), device="cuda", generator=gen)
    say("max_pool over 2.4e9 elements: backward")
    gx = K.max_pool2d_grad(gy, am, taps, tuple(x.shape), 2, 0, 2)
    want = torch.zeros_like(x).view(B, C, -1).scatter_add_(2, tidx.view(B, C, -1), gy.view(B, C, -1)).view_as(x)
    assert torch.equal(gx, want)
    del x, y, am, taps, tidx, gy, gx, want
    torch.cuda.empty_cache()


def test_reductions_and_elementwise_over_more_than_2_pow_31_elements(K):
    # [1500, 128, 112, 112] = 2.4e9 small integers: every partial sum stays below 2^24 in magnitude, so the sums are
    # exact in any order and must equal torch's (f64 where torch's own f32 order could round); the elementwise
    # kernels must reach the last element
    B, C, H, W = 1500, 128, 112, 112
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    x = torch.randint(-3, 4, (B, C, H, W), device="cuda", generator=gen).float()
    say("reductions over 2.4e9 elements")
    assert torch.equal(K.reduce_sum(x, [2, 3]), x.sum(dim=(2, 3)))
    assert torch.equal(K.reduce_sum(x, [0]), x.sum(dim=0))
    assert torch.equal(K.reduce_sum(x, [0, 2, 3]), x.double().sum(dim=(0, 2, 3)).float())
    assert torch.equal(K.reduce_mean(x, [1], True), x.mean(dim=1, keepdim=True))
    assert float(K.sum_all(x)) == float(x.double().sum())
    say("elementwise over 2.4e9 elements")
    b = torch.randint(-3, 4, (1, C, 1, 1), device="cuda", generator=gen).float()
    assert torch.equal(K.relu(x), torch.relu(x))
    assert torch.equal(K.add_broadcast_relu(x, b), torch.relu(x + b))
    assert torch.equal(K.broadcast_grad(b, tuple(x.shape), [0, 2, 3]), b.expand_as(x))
    del x
    torch.cuda.empty_cache()


def test_matmul_with_an_operand_of_more_than_2_pow_31_elements(K):
    # a [70000, 32768] operand (2.29e9 elements, past the kernels' 32-bit tile offsets) on either side and in either
    # storage order: the library cuts such a product along the big operand's rows where those are output rows or
    # columns, else along k.  Small integers, so every result is exact whatever the order of the sums.
    big, kk, small = 70000, 32768, 64
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4)
    X = torch.randint(-2, 3, (big, kk), device="cuda", generator=gen).float()
    S = torch.randint(-2, 3, (kk, small), device="cuda", generator=gen).float()
    St = S.t().contiguous()
    assert X.numel() > 2**31
    say("matmul, 2.29e9-element A [M,K]: rows cut")
    assert torch.equal(K.matmul(X, S), X @ S)
    say("matmul, 2.29e9-element B [N,K] transposed: columns cut")
    assert torch.equal(K.matmul(St, X, False, True), St @ X.t())
    Xt = X.t().contiguous()
    del X
    say("matmul, 2.29e9-element A [K,M] transposed: k cut")
    assert torch.equal(K.matmul(Xt, S, True, False), Xt.t() @ S)
    say("matmul, 2.29e9-element B [K,N]: k cut")
    assert torch.equal(K.matmul(St, Xt), St @ Xt)
    del Xt
    torch.cuda.empty_cache()


def test_matmul_with_an_output_of_more_than_2_pow_31_elements(K):
    # [70000, 64] x [64, 32768]: 2.29e9 output elements through the direct-to-LDS kernel (k = 64) and, with k = 40,
    # through the register-staged one; small integers, exact
    M, N, kk = 70000, 32768, 64
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    A = torch.randint(-2, 3, (M, kk), device="cuda", generator=gen).float()
    B = torch.randint(-2, 3, (kk, N), device="cuda", generator=gen).float()
    ref = A @ B
    say("matmul with 2.29e9 output elements")
    assert torch.equal(K.matmul(A, B), ref)
    assert torch.equal(K.matmul(A.t().contiguous(), B, True, False), ref)
    del ref
    say("matmul with 2.29e9 output elements, k = 40")
    assert torch.equal(K.matmul(A[:, :40].contiguous(), B[:40].contiguous()), A[:, :40] @ B[:40])
    del A, B
    torch.cuda.empty_cache()
