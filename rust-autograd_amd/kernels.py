"""Eager launchers: each function allocates the outputs as torch CUDA tensors (torch is only the
owner of device memory and of the stream) and calls the matching C-ABI entry point of
libag_hip.so.  Names and argument order follow the reference's compute functions
(conv2d_impl, conv2d_filter_grad_impl, conv2d_transpose_impl, max_pool_f32, ...), so that the
parity tests read like the reference's own tests.
"""
import ctypes as C

import torch

from . import capi
from .capi import check


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _f32(t, name):
    if not (isinstance(t, torch.Tensor) and t.is_cuda):
        raise capi.TypeUnsupported(f"{name}: expected a CUDA tensor")
    if t.dtype != torch.float32:
        raise capi.TypeUnsupported(f"{name}: only f32 is supported on the GPU path")
    return t.contiguous()   # the reference deep-copies non-contiguous inputs (conv2d.rs:436-452)


def _empty(shape, like, dtype=torch.float32):
    return torch.empty(tuple(int(s) for s in shape), dtype=dtype, device=like.device)


def _ws(nbytes, like):
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=like.device)


def conv_out_size(x, k, p, s, d):
    return capi.lib().ag_conv_out_size(x, k, p, s, d)


# ------------------------------------------------------------------------------------------ im2col
def im2col(x, kh, kw, ph, pw, sh, sw, dh, dw):
    x = _f32(x, "im2col")
    B, Cc, H, W = x.shape
    OH, OW = conv_out_size(H, kh, ph, sh, dh), conv_out_size(W, kw, pw, sw, dw)
    cols = _empty((B, Cc * kh * kw, max(OH, 0) * max(OW, 0)), x)
    check(capi.lib().ag_im2col_f32(_stream(), _ptr(x), _ptr(cols), B, Cc, H, W, kh, kw, ph, pw, sh, sw, dh, dw))
    return cols


def col2im(cols, Cc, H, W, kh, kw, ph, pw, sh, sw, dh, dw, OH, OW):
    cols = _f32(cols, "col2im")
    B = cols.shape[0]
    gx = _empty((B, Cc, H, W), cols)
    check(capi.lib().ag_col2im_f32(_stream(), _ptr(cols), _ptr(gx), B, Cc, H, W, kh, kw, ph, pw, sh, sw, dh, dw,
                                   OH, OW))
    return gx


# ------------------------------------------------------------------------------------------ GEMM
def gemm(ta, tb, m, n, k, alpha, a, lda, stride_a, b, ldb, stride_b, beta, c, ldc, stride_c, batch):
    check(capi.lib().ag_gemm_f32(_stream(), int(ta), int(tb), m, n, k, alpha, _ptr(a), lda, stride_a, _ptr(b),
                                 ldb, stride_b, beta, _ptr(c), ldc, stride_c, batch))
    return c


def gemm_batchsum(ta, tb, m, n, k, alpha, a, lda, stride_a, b, ldb, stride_b, beta, c, ldc, batch):
    nbytes = capi.lib().ag_gemm_batchsum_f32_workspace(m, n, k, batch)
    ws = _ws(nbytes, c)
    check(capi.lib().ag_gemm_batchsum_f32(_stream(), int(ta), int(tb), m, n, k, alpha, _ptr(a), lda, stride_a,
                                          _ptr(b), ldb, stride_b, beta, _ptr(c), ldc, batch, _ptr(ws),
                                          ws.numel()))
    return c


def matmul(a, b, transpose_a=False, transpose_b=False):
    """MatMul::compute (dot_ops.rs:564-606)."""
    a, b = _f32(a, "matmul"), _f32(b, "matmul")
    if a.dim() != 2:
        raise capi.IncompatibleShape("lhs input for MatMul must be 2D")
    if b.dim() != 2:
        raise capi.IncompatibleShape("rhs input for MatMul must be 2D")
    m, k = (a.shape[1], a.shape[0]) if transpose_a else a.shape
    k2, n = (b.shape[1], b.shape[0]) if transpose_b else b.shape
    if k != k2:
        raise capi.IncompatibleShape(
            f"ndarray: inputs {m} × {k} and {k2} × {n} are not compatible for matrix multiplication")
    c = _empty((m, n), a)
    L = capi.lib()
    ws = _ws(L.ag_matmul_f32_workspace(m, n, k), a)
    check(L.ag_matmul_f32(_stream(), int(transpose_a), int(transpose_b), m, n, k, _ptr(a), max(a.shape[1], 1), _ptr(b),
                          max(b.shape[1], 1), _ptr(c), max(n, 1), _ptr(ws), ws.numel()))
    return c


def batch_matmul(a, b, transpose_a=False, transpose_b=False):
    """BatchMatMul::compute (dot_ops.rs:631-695)."""
    a, b = _f32(a, "batch_matmul"), _f32(b, "batch_matmul")
    if a.dim() < 2:
        raise capi.IncompatibleShape(f"BatchMatMul: Left-hand-side input's ndim must be >= 2, actual: {a.dim()}")
    if b.dim() < 2:
        raise capi.IncompatibleShape(f"BatchMatMul: Right-hand-side input's ndim must be >= 2, actual: {b.dim()}")
    sa = list(a.shape)
    sb = list(b.shape)
    if transpose_a:
        sa[-2], sa[-1] = sa[-1], sa[-2]
    if transpose_b:
        sb[-2], sb[-1] = sb[-1], sb[-2]
    if len(sa) != len(sb) or sa[:-2] != sb[:-2]:
        raise capi.IncompatibleShape(f"Input shapes mismatch: {sa} vs {sb}")
    m, k, k2, n = sa[-2], sa[-1], sb[-2], sb[-1]
    if k != k2:
        raise capi.IncompatibleShape(f"Input shapes mismatch: {sa} vs {sb}")
    batch = 1
    for s in sa[:-2]:
        batch *= s
    c = _empty(sa[:-2] + [m, n], a)
    return gemm(transpose_a, transpose_b, m, n, k, 1.0, a, max(a.shape[-1], 1), a.shape[-1] * a.shape[-2], b,
                max(b.shape[-1], 1), b.shape[-1] * b.shape[-2], 0.0, c, max(n, 1), m * n, batch)


# ------------------------------------------------------------------------------------------ conv
def conv2d(x, w, pad, stride, dilation=1):
    """Conv2D::compute: returns (y, cols), the op's two outputs (conv2d.rs:531-554)."""
    x, w = _f32(x, "conv2d"), _f32(w, "conv2d")
    if x.dim() != 4:
        raise capi.IncompatibleShape(f"conv2d: lhs input must be 4D (got {list(x.shape)})")
    if w.dim() != 4:
        raise capi.IncompatibleShape(f"conv2d: filter must be 4D (got {list(w.shape)})")
    B, Cc, H, W = x.shape
    K, C2, kh, kw = w.shape
    if Cc != C2:
        raise capi.IncompatibleShape(
            f"conv2d: input channel dim ({Cc}) must match filter's second dim ({C2})")
    OH, OW = conv_out_size(H, kh, pad, stride, dilation), conv_out_size(W, kw, pad, stride, dilation)
    y = _empty((B, K, max(OH, 0), max(OW, 0)), x)
    cols = _empty((B, Cc * kh * kw, max(OH, 0) * max(OW, 0)), x)
    check(capi.lib().ag_conv2d_fwd_f32(_stream(), _ptr(x), _ptr(w), _ptr(y), _ptr(cols), B, Cc, H, W, K, kh, kw,
                                       pad, stride, dilation))
    return y, cols


def conv2d_with_cols(cols, w, OH, OW):
    cols, w = _f32(cols, "conv2d_with_cols"), _f32(w, "conv2d_with_cols")
    B = cols.shape[0]
    K, CK = w.shape[0], w.shape[1] * w.shape[2] * w.shape[3]
    y = _empty((B, K, OH, OW), cols)
    check(capi.lib().ag_conv2d_with_cols_f32(_stream(), _ptr(cols), _ptr(w), _ptr(y), B, CK, OH * OW, K))
    return y


def conv2d_filter_grad(cols, gy, w_shape):
    """Conv2DFilterGrad::compute (conv2d.rs:736-744)."""
    cols, gy = _f32(cols, "conv2d_filter_grad"), _f32(gy, "conv2d_filter_grad")
    B, K, OH, OW = gy.shape
    CK = w_shape[1] * w_shape[2] * w_shape[3]
    gw = _empty(w_shape, gy)
    nbytes = capi.lib().ag_conv2d_filter_grad_f32_workspace(B, CK, OH * OW, K)
    ws = _ws(nbytes, gy)
    check(capi.lib().ag_conv2d_filter_grad_f32(_stream(), _ptr(cols), _ptr(gy), _ptr(gw), B, CK, OH * OW, K,
                                               _ptr(ws), ws.numel()))
    return gw


def conv2d_transpose(gy, w, pad, stride, dilation=1, out_hw=None, return_cols=False):
    """Conv2DTranspose::compute (conv2d_transpose.rs:249-272).  out_hw=None reproduces the
    reference's reconstructed output size (conv2d_transpose.rs:55-56)."""
    gy, w = _f32(gy, "conv2d_transpose"), _f32(w, "conv2d_transpose")
    if gy.dim() != 4:
        raise capi.IncompatibleShape(f"conv2d_transpose: Input must be 4D (got {list(gy.shape)})")
    if w.dim() != 4:
        raise capi.IncompatibleShape(f"conv2d_transpose: Filter must be 4D (got {list(w.shape)})")
    B, ych, yh, yw = gy.shape
    ych2, xch, kh, kw = w.shape
    if ych != ych2:
        raise capi.IncompatibleShape(
            f"conv2d_transpose: Number of input channels ({ych}) must match second filter dim ({ych2})")
    if out_hw is None:
        L = capi.lib()
        out_hw = (L.ag_conv_transpose_out_size(yh, kh, pad, stride, dilation),
                  L.ag_conv_transpose_out_size(yw, kw, pad, stride, dilation))
    xh, xw = out_hw
    gx = _empty((B, xch, xh, xw), gy)
    gcols = _empty((B, xch * kh * kw, yh * yw), gy)
    L = capi.lib()
    if return_cols:
        # the caller wants the columns: the reference's two steps through their own entry points, the GEMM
        # gcols_b = w^T . gy_b (conv2d_transpose.rs:114-116, 167-182) and col2im (conv_ops/mod.rs:178-223), with the
        # operator's argument checks done by a call on an empty batch
        check(L.ag_conv2d_transpose_f32(_stream(), _ptr(gy), _ptr(w), _ptr(gx), _ptr(gcols), 0, ych, yh, yw,
                                        xch, kh, kw, pad, stride, dilation, xh, xw))
        M, P = xch * kh * kw, yh * yw
        if B and M and P:
            check(L.ag_gemm_f32(_stream(), 1, 0, M, P, ych, 1.0, _ptr(w), M, 0, _ptr(gy), P, ych * P, 0.0, _ptr(gcols), P,
                                M * P, B))
        check(L.ag_col2im_f32(_stream(), _ptr(gcols), _ptr(gx), B, xch, xh, xw, kh, kw, pad, pad, stride, stride,
                              dilation, dilation, yh, yw))
        return gx, gcols
    check(L.ag_conv2d_transpose_f32(_stream(), _ptr(gy), _ptr(w), _ptr(gx), _ptr(gcols), B, ych, yh, yw,
                                    xch, kh, kw, pad, stride, dilation, xh, xw))
    return gx


def conv2d_nocols(x, w, pad, stride=1, dilation=1):
    """Column-free forward (stride 1 or 2): (y, xpad) or None when the geometry is not supported.
    `xpad` (the rearranged input) is what conv2d_filter_grad_nocols reads instead of the columns."""
    x, w = _f32(x, "conv2d"), _f32(w, "conv2d")
    B, Cc, H, W = x.shape
    Kf, C2, kh, kw = w.shape
    if Cc != C2:
        raise capi.IncompatibleShape(f"conv2d: Number of input channels ({Cc}) must match second filter dim ({C2})")
    L = capi.lib()
    n = L.ag_conv2d_nocols_scratch_floats(B, Cc, H, W, Kf, kh, kw, pad, stride, dilation)
    if n == 0:
        return None
    xpad = torch.empty(n, dtype=torch.float32, device=x.device)
    OH, OW = conv_out_size(H, kh, pad, stride, dilation), conv_out_size(W, kw, pad, stride, dilation)
    y = _empty((B, Kf, OH, OW), x)
    check(L.ag_conv2d_fwd_nocols_f32(_stream(), _ptr(x), _ptr(w), _ptr(y), _ptr(xpad), B, Cc, H, W, Kf, kh, kw, pad,
                                     stride, dilation))
    return y, xpad


def conv_input_grad_staged(gy, w, pad, x_hw, stride=1, dilation=1):
    """The two stages of the column-free input gradient (stride 1 or 2): (gx, scratch); the scratch
    starts with the zero-bordered gy that conv2d_filter_grad_nocols takes.  None when not supported."""
    gy, w = _f32(gy, "conv2d_transpose"), _f32(w, "conv2d_transpose")
    B, ych, yh, yw = gy.shape
    _, xch, kh, kw = w.shape
    xh, xw = x_hw
    L = capi.lib()
    geom = (B, ych, yh, yw, xch, kh, kw, pad, stride, dilation, xh, xw)
    n = L.ag_conv_input_grad_scratch_floats(*geom)
    if n == 0:
        return None
    scratch = torch.empty(n, dtype=torch.float32, device=gy.device)
    gx = _empty((B, xch, xh, xw), gy)
    check(L.ag_conv_input_grad_prepare_f32(_stream(), _ptr(gy), _ptr(w), _ptr(scratch), *geom))
    check(L.ag_conv_input_grad_gemm_f32(_stream(), _ptr(scratch), _ptr(gx), *geom))
    return gx, scratch


def conv2d_filter_grad_nocols(xpad, gypad, x_shape, w_shape, pad, stride=1, dilation=1):
    """Column-free filter gradient from the rearranged copies of x (conv2d_nocols) and gy
    (conv_input_grad_staged): "same" convolutions for stride 1, any supported geometry for stride 2."""
    B, Cc, H, W = x_shape
    Kf, _, kh, kw = w_shape
    L = capi.lib()
    gw = _empty(w_shape, xpad)
    geom = (B, Cc, H, W, Kf, kh, kw, pad, stride, dilation)
    ws = _ws(L.ag_conv2d_filter_grad_nocols_f32_workspace(*geom), xpad)
    check(L.ag_conv2d_filter_grad_nocols_f32(_stream(), _ptr(xpad), _ptr(gypad), _ptr(gw), *geom, _ptr(ws), ws.numel()))
    return gw


def conv2d_transpose_filter_grad(x, gy, w_shape, pad, stride, dilation=1):
    """Conv2DTransposeFilterGrad::compute (conv2d_transpose.rs:433-451)."""
    x, gy = _f32(x, "conv2d_transpose_filter_grad"), _f32(gy, "conv2d_transpose_filter_grad")
    B, ych, yh, yw = x.shape
    _, xch, H, W = gy.shape
    kh, kw = w_shape[2], w_shape[3]
    gw = _empty(w_shape, x)
    gycols = _empty((B, xch * kh * kw, yh * yw), x)
    nbytes = capi.lib().ag_conv2d_filter_grad_f32_workspace(B, xch * kh * kw, yh * yw, ych)
    ws = _ws(nbytes, x)
    check(capi.lib().ag_conv2d_transpose_filter_grad_f32(_stream(), _ptr(x), _ptr(gy), _ptr(gw), _ptr(gycols), B,
                                                         ych, yh, yw, xch, H, W, kh, kw, pad, stride, dilation,
                                                         _ptr(ws), ws.numel()))
    return gw


# ------------------------------------------------------------------------------------------ pooling
def max_pool2d(x, pool_size, pad, stride):
    """MaxPool2D::compute: returns (y, argmax as f32, tap bytes = exact selection inside each window)."""
    x = _f32(x, "max_pool2d")
    B, Cc, H, W = x.shape
    L = capi.lib()
    OH, OW = L.ag_pool_out_size(H, pool_size, pad, stride), L.ag_pool_out_size(W, pool_size, pad, stride)
    y = _empty((B, Cc, max(OH, 0), max(OW, 0)), x)
    am = torch.empty_like(y)
    il = torch.empty(y.shape, dtype=torch.uint8, device=x.device)
    check(L.ag_maxpool2d_fwd_f32(_stream(), _ptr(x), _ptr(y), _ptr(am), _ptr(il), B, Cc, H, W, pool_size, pad,
                                 stride))
    return y, am, il


def relu_max_pool2d(a, b=None):
    """relu(a) or relu(a + b) followed by max_pool2d(2, pad 0, stride 2) in one launch: (r, y, argmax, taps)."""
    a = _f32(a, "relu_max_pool2d")
    if a.dim() != 4:
        raise capi.IncompatibleShape(f"max_pool2d: input must be 4D (got {list(a.shape)})")
    B, Cc, H, W = a.shape
    r = torch.empty_like(a)
    y = _empty((B, Cc, H // 2, W // 2), a)
    am = torch.empty_like(y)
    taps = torch.empty(y.shape, dtype=torch.uint8, device=a.device)
    bshape = None
    if b is not None:
        b = _f32(b, "relu_max_pool2d")
        if b.dim() != 4:
            raise capi.IncompatibleShape(f"add: operands of rank 4 and {b.dim()}")
        bshape = (C.c_int * 4)(*b.shape)
    check(capi.lib().ag_relu_maxpool2d_2x2_f32(_stream(), _ptr(a), _ptr(b), bshape, _ptr(r), _ptr(y), _ptr(am), _ptr(taps),
                                               B, Cc, H, W))
    return r, y, am, taps


def max_pool2d_grad(gy, argmax, taps, x_shape, pool_size, pad, stride):
    gy = _f32(gy, "max_pool2d_grad")
    B, Cc, H, W = x_shape
    gx = _empty(x_shape, gy)
    check(capi.lib().ag_maxpool2d_bwd_f32(_stream(), _ptr(gy), _ptr(argmax), _ptr(taps), _ptr(gx), B, Cc, H,
                                          W, pool_size, pad, stride))
    return gx


def max_pool2d_grad_relu(gy, argmax, taps, relu_x, pool_size, pad, stride):
    """MaxPool2DGrad and the gradient of the ReLU in front of the pooling in one pass:
    greater(relu_x, 0) * max_pool2d_grad(gy)."""
    gy, relu_x = _f32(gy, "max_pool2d_grad"), _f32(relu_x, "max_pool2d_grad")
    B, Cc, H, W = relu_x.shape
    gx = _empty(tuple(relu_x.shape), gy)
    check(capi.lib().ag_maxpool2d_bwd_relu_f32(_stream(), _ptr(gy), _ptr(argmax), _ptr(taps), _ptr(relu_x), _ptr(gx),
                                               B, Cc, H, W, pool_size, pad, stride))
    return gx


def max_pool2d_grad_grad(ggx, argmax, taps, pool_size, pad, stride):
    ggx = _f32(ggx, "max_pool2d_grad_grad")
    B, Cc, H, W = ggx.shape
    L = capi.lib()
    OH, OW = L.ag_pool_out_size(H, pool_size, pad, stride), L.ag_pool_out_size(W, pool_size, pad, stride)
    ggy = _empty((B, Cc, OH, OW), ggx)
    check(L.ag_maxpool2d_gradgrad_f32(_stream(), _ptr(ggx), _ptr(argmax), _ptr(taps), _ptr(ggy), B, Cc, H, W,
                                      pool_size, pad, stride))
    return ggy


# ------------------------------------------------------------------------------------------ reductions
def sum_all(x):
    x = _f32(x, "sum_all")
    out = _empty((), x)
    ws = _ws(capi.lib().ag_sum_all_f32_workspace(x.numel()), x)
    check(capi.lib().ag_sum_all_f32(_stream(), _ptr(x), x.numel(), _ptr(out), _ptr(ws), ws.numel()))
    return out


def _axes(axes, rank):
    ax = [int(a) % rank if rank else int(a) for a in axes]
    return ax, (C.c_int * max(1, len(ax)))(*ax)


def reduce_sum(x, axes, keep_dims=False, mean=False):
    x = _f32(x, "reduce_sum")
    ax, cax = _axes(axes, x.dim())
    shape = (C.c_int * max(1, x.dim()))(*x.shape)
    red = set(ax)
    out_shape = [1 if i in red else s for i, s in enumerate(x.shape)]
    out = _empty(out_shape, x)
    L = capi.lib()
    ws = _ws(L.ag_reduce_sum_f32_workspace(shape, x.dim(), cax, len(ax)), x)
    check(L.ag_reduce_sum_f32(_stream(), _ptr(x), _ptr(out), shape, x.dim(), cax, len(ax), int(mean), _ptr(ws),
                              ws.numel()))
    if not keep_dims:
        out = out.reshape([s for i, s in enumerate(x.shape) if i not in red])
    return out


def reduce_mean(x, axes, keep_dims=False):
    return reduce_sum(x, axes, keep_dims, mean=True)


def broadcast_grad(gy, x_shape, axes):
    gy = _f32(gy, "reduce_grad")
    rank = len(x_shape)
    ax, cax = _axes(axes, rank)
    shape = (C.c_int * max(1, rank))(*x_shape)
    gx = _empty(x_shape, gy)
    check(capi.lib().ag_broadcast_grad_f32(_stream(), _ptr(gy), _ptr(gx), shape, rank, cax, len(ax)))
    return gx


# ------------------------------------------------------------------------------------------ Adam + glue
def adam_update(param, grad, m, v, t, alpha=1e-3, eps=1e-8, b1=0.9, b2=0.999):
    """AdamOp::compute: in place on param, m, v and the one-element step counter t."""
    for a in (param, grad, m, v, t):
        assert a.is_cuda and a.dtype == torch.float32 and a.is_contiguous()
    check(capi.lib().ag_adam_update_f32(_stream(), _ptr(param), _ptr(grad), _ptr(m), _ptr(v), _ptr(t),
                                        param.numel(), alpha, eps, b1, b2))


def adam_update_multi(params, grads, ms, vs, ts, alpha=1e-3, eps=1e-8, b1=0.9, b2=0.999):
    """One optimizer step over several parameters (one AdamOp::compute each in the reference) as one launch."""
    import ctypes as C
    n = len(params)
    assert len(grads) == len(ms) == len(vs) == len(ts) == n
    for a in (*params, *grads, *ms, *vs, *ts):
        assert a.is_cuda and a.dtype == torch.float32 and a.is_contiguous()
    table = lambda xs: (C.c_void_p * max(n, 1))(*[x.data_ptr() for x in xs])
    sizes = (C.c_size_t * max(n, 1))(*[p.numel() for p in params])
    check(capi.lib().ag_adam_update_multi_f32(_stream(), n, table(params), table(grads), table(ms), table(vs), table(ts),
                                              sizes, alpha, eps, b1, b2))


def relu(x):
    x = _f32(x, "relu")
    y = torch.empty_like(x)
    check(capi.lib().ag_relu_f32(_stream(), _ptr(x), _ptr(y), x.numel()))
    return y


def relu_grad(x, gy):
    x, gy = _f32(x, "relu_grad"), _f32(gy, "relu_grad")
    gx = torch.empty_like(x)
    check(capi.lib().ag_relu_grad_f32(_stream(), _ptr(x), _ptr(gy), _ptr(gx), x.numel()))
    return gx


def add_bias(x, bias):
    x, bias = _f32(x, "add"), _f32(bias, "add")
    y = torch.empty_like(x)
    check(capi.lib().ag_add_bias_f32(_stream(), _ptr(x), _ptr(bias), _ptr(y), x.shape[0], x.shape[1]))
    return y


def add_broadcast(x, b):
    """x + b where b has x's rank and extent 1 on the axes it is broadcast along."""
    x, b = _f32(x, "add"), _f32(b, "add")
    if x.dim() != b.dim():
        raise capi.IncompatibleShape(f"add: operands of rank {x.dim()} and {b.dim()}")
    y = torch.empty_like(x)
    shape = (C.c_int * max(x.dim(), 1))(*x.shape)
    bshape = (C.c_int * max(x.dim(), 1))(*b.shape)
    check(capi.lib().ag_add_broadcast_f32(_stream(), _ptr(x), _ptr(b), _ptr(y), shape, bshape, x.dim()))
    return y


def add_broadcast_relu(x, b):
    """relu(x + b) in one pass, b as for add_broadcast."""
    x, b = _f32(x, "add+relu"), _f32(b, "add+relu")
    if x.dim() != b.dim():
        raise capi.IncompatibleShape(f"add+relu: operands of rank {x.dim()} and {b.dim()}")
    y = torch.empty_like(x)
    shape = (C.c_int * max(x.dim(), 1))(*x.shape)
    bshape = (C.c_int * max(x.dim(), 1))(*b.shape)
    check(capi.lib().ag_add_broadcast_relu_f32(_stream(), _ptr(x), _ptr(b), _ptr(y), shape, bshape, x.dim()))
    return y


def bias_grad(gy):
    gy = _f32(gy, "reduce_sum")
    out = _empty((1, gy.shape[1]), gy)
    check(capi.lib().ag_bias_grad_f32(_stream(), _ptr(gy), _ptr(out), gy.shape[0], gy.shape[1]))
    return out


def add_n(xs):
    xs = [_f32(a, "add_n") for a in xs]
    out = torch.empty_like(xs[0])
    arr = (C.c_void_p * len(xs))(*[a.data_ptr() for a in xs])
    check(capi.lib().ag_add_n_f32(_stream(), arr, len(xs), _ptr(out), out.numel()))
    return out


def mul(a, b):
    a, b = _f32(a, "mul"), _f32(b, "mul")
    out = torch.empty_like(a)
    check(capi.lib().ag_mul_f32(_stream(), _ptr(a), _ptr(b), _ptr(out), a.numel()))
    return out


def scale(a, s):
    a = _f32(a, "scale")
    out = torch.empty_like(a)
    check(capi.lib().ag_scale_f32(_stream(), _ptr(a), float(s), _ptr(out), a.numel()))
    return out


def fill(shape, value, device="cuda"):
    out = torch.empty(tuple(shape), dtype=torch.float32, device=device)
    check(capi.lib().ag_fill_f32(_stream(), _ptr(out), float(value), out.numel()))
    return out


def sparse_softmax_cross_entropy(logits, labels):
    logits, labels = _f32(logits, "SparseSoftmaxCrossEntropy"), _f32(labels, "SparseSoftmaxCrossEntropy")
    if logits.dim() != 2:
        raise capi.IncompatibleShape(
            f"SparseSoftmaxCrossEntropy: given first argument's ndim is not 2: shape={list(logits.shape)}")
    if not (labels.dim() == 1 or (labels.dim() == 2 and labels.shape[1] == 1)):
        raise capi.IncompatibleShape(
            "SparseSoftmaxCrossEntropy: second argument's shape must be (batch_size, 1) or (batch_size,). "
            f"given shape={list(labels.shape)}")
    rows, classes = logits.shape
    loss = _empty((rows, 1), logits)
    lsm = torch.empty_like(logits)
    check(capi.lib().ag_sparse_softmax_xent_f32(_stream(), _ptr(logits), _ptr(labels), _ptr(loss), _ptr(lsm), rows,
                                                classes))
    return loss, lsm


def sparse_softmax_cross_entropy_grad(log_softmax, labels, gy):
    lsm, labels, gy = (_f32(log_softmax, "SparseSoftmaxCrossEntropyGrad"),
                       _f32(labels, "SparseSoftmaxCrossEntropyGrad"), _f32(gy, "SparseSoftmaxCrossEntropyGrad"))
    gx = torch.empty_like(lsm)
    check(capi.lib().ag_sparse_softmax_xent_grad_f32(_stream(), _ptr(lsm), _ptr(labels), _ptr(gy), _ptr(gx),
                                                     lsm.shape[0], lsm.shape[1]))
    return gx


def sparse_softmax_cross_entropy_grad_from_logits(logits, labels, gy):
    """The gradient without the forward's log-softmax; `gy`: a tensor of one value per row, or a float."""
    logits, labels = _f32(logits, "SparseSoftmaxCrossEntropyGrad"), _f32(labels, "SparseSoftmaxCrossEntropyGrad")
    gx = torch.empty_like(logits)
    const = isinstance(gy, (int, float))
    check(capi.lib().ag_sparse_softmax_xent_grad_logits_f32(_stream(), _ptr(logits), _ptr(labels), None if const else _ptr(gy),
                                                            float(gy) if const else 0.0, _ptr(gx), logits.shape[0], logits.shape[1]))
    return gx
