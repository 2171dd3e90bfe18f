"""ctypes front-end of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only the test-suite, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` import this module; the GPU library never does.  Every function
takes and returns numpy arrays and forwards to ``libag_oracle.so`` (built by
``oracle/Makefile`` from ``ag_oracle.c``), whose functions cite the reference
sources they restate.
"""
import ctypes as C
import glob
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libag_oracle.so")


def build(force=False):
    """Compile the oracle with gcc (a few seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libag_oracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_blas_name.restype = C.c_char_p
        _lib.orc_sum_all_f32.restype = C.c_float
        _lib.orc_sum_all_f64.restype = C.c_double
        _lib.orc_maxpool2d_bwd_f32.restype = C.c_long
        _lib.orc_maxpool2d_bwd_f64.restype = C.c_long
    return _lib


def _suf(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32", C.c_float
    if dtype == np.float64:
        return "f64", C.c_double
    raise TypeError("oracle supports float32 and float64 only")


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype=None):
    return np.ascontiguousarray(a, dtype=dtype)


def _fn(name, dtype):
    suf, real = _suf(dtype)
    return getattr(lib(), f"{name}_{suf}"), real


# --------------------------------------------------------------------------
# optional OpenBLAS for the timed baseline
# --------------------------------------------------------------------------
def load_openblas():
    """Try to load an OpenBLAS (system one, else SciPy's bundled copy).  Returns its path or None."""
    cands = []
    for pat in ("/usr/lib/x86_64-linux-gnu/libopenblas.so*", "/usr/lib64/libopenblas.so*",
                "/usr/lib/libopenblas.so*"):
        cands += sorted(glob.glob(pat))
    try:
        import scipy
        cands += sorted(glob.glob(os.path.join(os.path.dirname(scipy.__file__), "..", "scipy.libs",
                                               "libscipy_openblas-*.so")))
    except Exception:
        pass
    for c in cands:
        if lib().orc_blas_load(os.path.realpath(c).encode()):
            return os.path.realpath(c)
    return None


def unload_blas():
    lib().orc_blas_unload()


def blas_name():
    return lib().orc_blas_name().decode()


def blas_set_threads(n):
    lib().orc_blas_set_threads(int(n))


# --------------------------------------------------------------------------
# geometry helpers
# --------------------------------------------------------------------------
def conv_out_size(x, k, p, s, d):
    return lib().orc_conv_out_size(x, k, p, s, d)


def conv_transpose_out_size(y, k, p, s, d):
    return lib().orc_conv_transpose_out_size(y, k, p, s, d)


def pool_grad_in_size(y, size, p, s):
    return lib().orc_pool_grad_in_size(y, size, p, s)


# --------------------------------------------------------------------------
# im2col / col2im
# --------------------------------------------------------------------------
def im2col(x, kh, kw, ph, pw, sh, sw, dh, dw, literal_pad=True, threads=1):
    x = _c(x)
    B, Cc, H, W = x.shape
    OH, OW = conv_out_size(H, kh, ph, sh, dh), conv_out_size(W, kw, pw, sw, dw)
    cols = np.empty((B, Cc * kh * kw, OH * OW), dtype=x.dtype)
    f, _ = _fn("orc_im2col", x.dtype)
    f(_p(x), _p(cols), B, Cc, H, W, kh, kw, ph, pw, sh, sw, dh, dw, int(literal_pad), threads)
    return cols


def col2im(cols, Cc, H, W, kh, kw, ph, pw, sh, sw, dh, dw, OH, OW, threads=1):
    cols = _c(cols)
    B = cols.shape[0]
    assert cols.size == B * Cc * kh * kw * OH * OW
    gx = np.empty((B, Cc, H, W), dtype=cols.dtype)
    f, _ = _fn("orc_col2im", cols.dtype)
    f(_p(cols), _p(gx), B, Cc, H, W, kh, kw, ph, pw, sh, sw, dh, dw, OH, OW, threads)
    return gx


# --------------------------------------------------------------------------
# GEMM family
# --------------------------------------------------------------------------
def gemm(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, naive=False):
    f, real = _fn("orc_gemm_naive" if naive else "orc_gemm", c.dtype)
    f(int(ta), int(tb), m, n, k, real(alpha), _p(a), lda, _p(b), ldb, real(beta), _p(c), ldc)
    return c


def matmul(a, b, ta=False, tb=False):
    a, b = _c(a), _c(b)
    m, k = (a.shape[1], a.shape[0]) if ta else a.shape
    k2, n = (b.shape[1], b.shape[0]) if tb else b.shape
    assert k == k2
    c = np.empty((m, n), dtype=a.dtype)
    f, _ = _fn("orc_matmul", a.dtype)
    f(_p(a), _p(b), _p(c), m, n, k, int(ta), int(tb))
    return c


def batch_matmul(a, b, ta=False, tb=False, threads=1):
    a, b = _c(a), _c(b)
    lead = a.shape[:-2]
    batch = int(np.prod(lead)) if lead else 1
    m, k = (a.shape[-1], a.shape[-2]) if ta else a.shape[-2:]
    k2, n = (b.shape[-1], b.shape[-2]) if tb else b.shape[-2:]
    assert k == k2 and b.shape[:-2] == lead
    c = np.empty(lead + (m, n), dtype=a.dtype)
    f, _ = _fn("orc_batch_matmul", a.dtype)
    f(_p(a), _p(b), _p(c), batch, m, n, k, int(ta), int(tb), threads)
    return c


# --------------------------------------------------------------------------
# convolution ops
# --------------------------------------------------------------------------
def conv2d_fwd(x, w, pad, stride, dil, threads=1):
    """Returns (y [B,K,OH,OW], cols [B, C*kh*kw, OH*OW])."""
    x, w = _c(x), _c(w)
    B, Cc, H, W = x.shape
    K, C2, kh, kw = w.shape
    assert Cc == C2
    OH, OW = conv_out_size(H, kh, pad, stride, dil), conv_out_size(W, kw, pad, stride, dil)
    y = np.empty((B, K, OH, OW), dtype=x.dtype)
    cols = np.empty((B, Cc * kh * kw, OH * OW), dtype=x.dtype)
    f, _ = _fn("orc_conv2d_fwd", x.dtype)
    f(_p(x), _p(w), _p(y), _p(cols), B, Cc, H, W, K, kh, kw, pad, stride, dil, threads)
    return y, cols


def conv2d_with_cols(cols, w, OH, OW, threads=1):
    cols, w = _c(cols), _c(w)
    B = cols.shape[0]
    K = w.shape[0]
    CK = w.shape[1] * w.shape[2] * w.shape[3]
    y = np.empty((B, K, OH, OW), dtype=cols.dtype)
    f, _ = _fn("orc_conv2d_with_cols", cols.dtype)
    f(_p(cols), _p(w), _p(y), B, CK, OH * OW, K, threads)
    return y


def conv2d_filter_grad(cols, gy, w_shape):
    cols, gy = _c(cols), _c(gy)
    B, K, OH, OW = gy.shape
    CK = w_shape[1] * w_shape[2] * w_shape[3]
    gw = np.empty(tuple(w_shape), dtype=gy.dtype)
    f, _ = _fn("orc_conv2d_filter_grad", gy.dtype)
    f(_p(cols), _p(gy), _p(gw), B, CK, OH * OW, K)
    return gw


def conv2d_transpose(gy, w, pad, stride, dil, out_hw=None, threads=1, return_cols=False):
    """Conv2DTranspose.  out_hw=None uses the reference's reconstructed size."""
    gy, w = _c(gy), _c(w)
    B, ych, yh, yw = gy.shape
    ych2, xch, kh, kw = w.shape
    assert ych == ych2
    if out_hw is None:
        out_hw = (conv_transpose_out_size(yh, kh, pad, stride, dil),
                  conv_transpose_out_size(yw, kw, pad, stride, dil))
    xh, xw = out_hw
    gx = np.empty((B, xch, xh, xw), dtype=gy.dtype)
    gcols = np.empty((B, xch * kh * kw, yh * yw), dtype=gy.dtype)
    f, _ = _fn("orc_conv2d_transpose", gy.dtype)
    f(_p(gy), _p(w), _p(gx), _p(gcols), B, ych, yh, yw, xch, kh, kw, pad, stride, dil, xh, xw, threads)
    return (gx, gcols) if return_cols else gx


def conv2d_transpose_filter_grad(x, gy, w_shape, pad, stride, dil, threads=1):
    """x [B,ych,yh,yw] (input of the transposed conv), gy [B,xch,H,W] (grad of its output)."""
    x, gy = _c(x), _c(gy)
    B, ych, yh, yw = x.shape
    _, xch, H, W = gy.shape
    kh, kw = w_shape[2], w_shape[3]
    assert conv_out_size(H, kh, pad, stride, dil) == yh and conv_out_size(W, kw, pad, stride, dil) == yw
    gw = np.empty(tuple(w_shape), dtype=x.dtype)
    gycols = np.empty((B, xch * kh * kw, yh * yw), dtype=x.dtype)
    f, _ = _fn("orc_conv2d_transpose_filter_grad", x.dtype)
    f(_p(x), _p(gy), _p(gw), _p(gycols), B, ych, yh, yw, xch, H, W, kh, kw, pad, stride, dil, threads)
    return gw


# --------------------------------------------------------------------------
# max pooling
# --------------------------------------------------------------------------
def maxpool2d_fwd(x, size, pad, stride):
    """Returns (y, argmax stored as x.dtype, exact plane-local int32 index)."""
    x = _c(x)
    B, Cc, H, W = x.shape
    OH, OW = (H + 2 * pad - size) // stride + 1, (W + 2 * pad - size) // stride + 1
    y = np.empty((B, Cc, OH, OW), dtype=x.dtype)
    am = np.empty_like(y)
    il = np.empty(y.shape, dtype=np.int32)
    f, _ = _fn("orc_maxpool2d_fwd", x.dtype)
    rc = f(_p(x), _p(y), _p(am), _p(il), B, Cc, H, W, size, pad, stride)
    if rc != 0:
        raise ValueError("max_pool2d: pad must be 0")
    return y, am, il


def maxpool2d_taps(idx_local, W, size, stride):
    """The exact selection as one byte per output: dy*size + dx of the selected pixel inside its
    window, 255 where idx_local is -1 (derived from the plane-local index the oracle returns)."""
    il = np.asarray(idx_local, dtype=np.int64)
    OH, OW = il.shape[-2:]
    oy = np.arange(OH).reshape(-1, 1)
    ox = np.arange(OW).reshape(1, -1)
    tap = (il // W - oy * stride) * size + (il % W - ox * stride)
    return np.where(il >= 0, tap, 255).astype(np.uint8)


def maxpool2d_bwd(gy, argmax, x_shape):
    gy, argmax = _c(gy), _c(argmax, gy.dtype)
    gx = np.empty(tuple(x_shape), dtype=gy.dtype)
    f, _ = _fn("orc_maxpool2d_bwd", gy.dtype)
    skipped = f(_p(gy), _p(argmax), _p(gx), C.c_size_t(gy.size), C.c_size_t(gx.size))
    return gx, int(skipped)


def maxpool2d_bwd_local(gy, idx_local, x_shape):
    gy, idx_local = _c(gy), _c(idx_local, np.int32)
    B, Cc, H, W = x_shape
    gx = np.empty(tuple(x_shape), dtype=gy.dtype)
    f, _ = _fn("orc_maxpool2d_bwd_local", gy.dtype)
    f(_p(gy), _p(idx_local), _p(gx), C.c_size_t(B * Cc), C.c_size_t(gy.shape[2] * gy.shape[3]),
      C.c_size_t(H * W))
    return gx


def maxpool2d_gradgrad(ggx, argmax, y_shape):
    ggx, argmax = _c(ggx), _c(argmax, ggx.dtype)
    ggy = np.empty(tuple(y_shape), dtype=ggx.dtype)
    f, _ = _fn("orc_maxpool2d_gradgrad", ggx.dtype)
    f(_p(ggx), _p(argmax), _p(ggy), C.c_size_t(ggy.size), C.c_size_t(ggx.size))
    return ggy


# --------------------------------------------------------------------------
# reductions
# --------------------------------------------------------------------------
def sum_all(x):
    x = _c(x)
    f, _ = _fn("orc_sum_all", x.dtype)
    return x.dtype.type(f(_p(x), C.c_size_t(x.size)))


def _axes(axes, rank):
    ax = sorted({int(a) % rank for a in axes})
    return ax, (C.c_int * max(1, len(ax)))(*ax)


def reduce_sum(x, axes, keep_dims=False, mean=False):
    x = _c(x)
    ax, cax = _axes(axes, x.ndim)
    shape = (C.c_int * x.ndim)(*x.shape)
    out_shape = [1 if i in ax else s for i, s in enumerate(x.shape)]
    out = np.empty(out_shape, dtype=x.dtype)
    f, _ = _fn("orc_reduce_sum", x.dtype)
    f(_p(x), _p(out), shape, x.ndim, cax, len(ax), int(mean))
    if not keep_dims:
        out = out.reshape([s for i, s in enumerate(x.shape) if i not in ax])
    return out


def reduce_mean(x, axes, keep_dims=False):
    return reduce_sum(x, axes, keep_dims, mean=True)


def broadcast_grad(gy, x_shape, axes):
    gy = _c(gy)
    rank = len(x_shape)
    ax, cax = _axes(axes, rank)
    shape = (C.c_int * rank)(*x_shape)
    gx = np.empty(tuple(x_shape), dtype=gy.dtype)
    f, _ = _fn("orc_broadcast_grad", gy.dtype)
    f(_p(gy), _p(gx), shape, rank, cax, len(ax))
    return gx


# --------------------------------------------------------------------------
# Adam and glue
# --------------------------------------------------------------------------
def adam(p, g, m, v, t, alpha=1e-3, eps=1e-8, b1=0.9, b2=0.999):
    """In place on p, m, v, t (t is a 1-element array), like AdamOp."""
    assert all(a.flags.c_contiguous for a in (p, g, m, v, t))
    f, real = _fn("orc_adam", p.dtype)
    f(_p(p), _p(g), _p(m), _p(v), _p(t), C.c_size_t(p.size), real(alpha), real(eps), real(b1), real(b2))


def relu(x):
    x = _c(x)
    y = np.empty_like(x)
    f, _ = _fn("orc_relu", x.dtype)
    f(_p(x), _p(y), C.c_size_t(x.size))
    return y


def relu_grad(x, gy):
    x, gy = _c(x), _c(gy)
    gx = np.empty_like(x)
    f, _ = _fn("orc_relu_grad", x.dtype)
    f(_p(x), _p(gy), _p(gx), C.c_size_t(x.size))
    return gx


def add_bias(x, bias):
    x, bias = _c(x), _c(bias)
    y = np.empty_like(x)
    f, _ = _fn("orc_add_bias", x.dtype)
    f(_p(x), _p(bias), _p(y), C.c_size_t(x.shape[0]), C.c_size_t(x.shape[1]))
    return y


def add_n(xs):
    xs = [_c(a) for a in xs]
    out = np.empty_like(xs[0])
    arr = (C.c_void_p * len(xs))(*[a.ctypes.data for a in xs])
    f, _ = _fn("orc_add_n", out.dtype)
    f(arr, len(xs), _p(out), C.c_size_t(out.size))
    return out


def sparse_softmax_xent(logits, labels):
    logits = _c(logits)
    labels = _c(labels, logits.dtype).reshape(-1)
    rows, classes = logits.shape
    loss = np.empty((rows, 1), dtype=logits.dtype)
    lsm = np.empty_like(logits)
    f, _ = _fn("orc_sparse_softmax_xent", logits.dtype)
    f(_p(logits), _p(labels), _p(loss), _p(lsm), C.c_size_t(rows), C.c_size_t(classes))
    return loss, lsm


def sparse_softmax_xent_grad(log_softmax, labels, gy):
    lsm = _c(log_softmax)
    labels = _c(labels, lsm.dtype).reshape(-1)
    gy = _c(gy, lsm.dtype).reshape(-1)
    gx = np.empty_like(lsm)
    f, _ = _fn("orc_sparse_softmax_xent_grad", lsm.dtype)
    f(_p(lsm), _p(labels), _p(gy), _p(gx), C.c_size_t(lsm.shape[0]), C.c_size_t(lsm.shape[1]))
    return gx
