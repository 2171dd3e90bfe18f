"""The convolution and its two gradients by their definitions, in f64, on sampled output elements:
the host truth of the full-size GPU tests (the f64 oracle itself would need the 1.85 GB x 2 of
columns in f64).  tests/test_oracle.py checks these against the oracle on small cases."""
import numpy as np


def direct_y(x, w, idx, pad, stride, dil):
    """y[b,k,oy,ox] by the definition, f64, for the sampled (b,k,oy,ox) rows of idx."""
    Kf, C, kh, kw = w.shape
    H, W = x.shape[2:]
    b, k, oy, ox = idx.T
    out = np.zeros(len(idx))
    w64 = w.astype(np.float64)
    for ky in range(kh):
        for kx in range(kw):
            iy, ix = oy * stride - pad + ky * dil, ox * stride - pad + kx * dil
            ok = (iy >= 0) & (iy < H) & (ix >= 0) & (ix < W)
            patch = x[b[ok], :, iy[ok], ix[ok]].astype(np.float64)            # [n, C]
            out[ok] += np.einsum("nc,nc->n", patch, w64[k[ok], :, ky, kx])
    return out


def direct_gx(gy, w, idx, pad, stride, dil):
    """gx[b,c,iy,ix] = sum over filters and taps of gy[b,k,oy,ox] w[k,c,ky,kx] with
    oy*stride - pad + ky*dil == iy (conv_ops/mod.rs:178-223 after the GEMM of conv2d_transpose.rs:167-182)."""
    Kf, C, kh, kw = w.shape
    OH, OW = gy.shape[2:]
    b, c, iy, ix = idx.T
    out = np.zeros(len(idx))
    w64 = w.astype(np.float64)
    for ky in range(kh):
        for kx in range(kw):
            ny, nx = iy + pad - ky * dil, ix + pad - kx * dil
            oy, ox = ny // stride, nx // stride
            ok = (ny % stride == 0) & (nx % stride == 0) & (oy >= 0) & (oy < OH) & (ox >= 0) & (ox < OW)
            g = gy[b[ok], :, oy[ok], ox[ok]].astype(np.float64)               # [n, Kf]
            out[ok] += np.einsum("nk,nk->n", g, w64[:, c[ok], ky, kx].T)
    return out


def direct_gw(x, gy, chans, kh, kw, pad, stride, dil):
    """gw[:, chans, :, :] = sum over images and positions of gy[b,k,oy,ox] x[b,c,iy,ix], f64 (dgemm per tap)."""
    B, C, H, W = x.shape
    _, Kf, OH, OW = gy.shape
    xp = np.zeros((B, len(chans), H + 2 * pad, W + 2 * pad), np.float64)
    xp[:, :, pad:pad + H, pad:pad + W] = x[:, chans]
    g2 = gy.astype(np.float64).transpose(1, 0, 2, 3).reshape(Kf, B * OH * OW)
    out = np.zeros((Kf, len(chans), kh, kw))
    for ky in range(kh):
        for kx in range(kw):
            tap = xp[:, :, ky * dil:ky * dil + stride * (OH - 1) + 1:stride, kx * dil:kx * dil + stride * (OW - 1) + 1:stride]
            out[:, :, ky, kx] = g2 @ tap.transpose(0, 2, 3, 1).reshape(B * OH * OW, len(chans))
    return out
