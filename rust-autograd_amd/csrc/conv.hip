// Convolution operators as compositions of im2col / col2im and the MFMA GEMM, mirroring how the
// reference builds them (conv2d.rs:25-112, 631-734; conv2d_transpose.rs:89-247, 303-431) but
// batched: one im2col launch and one strided-batched GEMM launch per operator instead of one
// task per image, and one split-accumulation GEMM instead of an image-sequential beta=1 loop.
#include "ag_internal.h"

using namespace ag;

static ag_status_t conv_dims(const char *who, int B, int C, int H, int W, int K, int kh, int kw, int pad,
                             int stride, int dilation)
{
    AG_REQUIRE(B >= 0 && C >= 0 && H >= 0 && W >= 0 && K >= 0, AG_ERR_INVALID_DIMS,
               "%s: negative extent (B=%d C=%d H=%d W=%d K=%d)", who, B, C, H, W, K);
    AG_REQUIRE(kh >= 1 && kw >= 1 && stride >= 1 && dilation >= 1 && pad >= 0, AG_ERR_INVALID_DIMS,
               "%s: kernel/stride/dilation must be >= 1 and pad >= 0 (k=%dx%d stride=%d dilation=%d pad=%d)", who,
               kh, kw, stride, dilation, pad);
    return AG_OK;
}

extern "C" ag_status_t ag_conv2d_fwd_f32(ag_stream_t stream, const float *x, const float *w, float *y,
                                         float *cols, int B, int C, int H, int W, int K, int kh, int kw,
                                         int pad, int stride, int dilation)
{
    if (ag_status_t s = conv_dims("conv2d", B, C, H, W, K, kh, kw, pad, stride, dilation)) return s;
    AG_REQUIRE(H + 2 * pad >= dilation * (kh - 1) + 1 && W + 2 * pad >= dilation * (kw - 1) + 1,
               AG_ERR_INCOMPATIBLE_SHAPE, "conv2d: filter extent exceeds the padded input (%dx%d)", H, W);
    const int OH = ag_conv_out_size(H, kh, pad, stride, dilation);
    const int OW = ag_conv_out_size(W, kw, pad, stride, dilation);
    const long long CK = (long long)C * kh * kw, P = (long long)OH * OW;
    AG_REQUIRE(CK <= 0x7fffffff && P <= 0x7fffffff, AG_ERR_INVALID_DIMS, "conv2d: matrix extent overflows int");
    if (ag_status_t s = ag_im2col_f32(stream, x, cols, B, C, H, W, kh, kw, pad, pad, stride, stride, dilation,
                                      dilation))
        return s;
    return ag_gemm_f32(stream, 0, 0, K, (int)P, (int)CK, 1.f, w, (int)CK, 0, cols, (int)P, CK * P, 0.f, y,
                       (int)P, (long long)K * P, B);
}

extern "C" ag_status_t ag_conv2d_with_cols_f32(ag_stream_t stream, const float *cols, const float *w,
                                               float *y, int B, int CK, int P, int K)
{
    return ag_gemm_f32(stream, 0, 0, K, P, CK, 1.f, w, CK, 0, cols, P, (long long)CK * P, 0.f, y, P,
                       (long long)K * P, B);
}

extern "C" size_t ag_conv2d_filter_grad_f32_workspace(int B, int CK, int P, int K)
{
    return ag_gemm_batchsum_f32_workspace(K, CK, P, B);
}

extern "C" ag_status_t ag_conv2d_filter_grad_f32(ag_stream_t stream, const float *cols, const float *gy,
                                                 float *gw, int B, int CK, int P, int K, void *ws,
                                                 size_t ws_bytes)
{
    // gw[K x CK] = sum_b gy_b[K x P] * cols_b[CK x P]^T        conv2d.rs:662-687
    return ag_gemm_batchsum_f32(stream, 0, 1, K, CK, P, 1.f, gy, P, (long long)K * P, cols, P,
                                (long long)CK * P, 0.f, gw, CK, B, ws, ws_bytes);
}

extern "C" ag_status_t ag_conv2d_transpose_f32(ag_stream_t stream, const float *gy, const float *w,
                                               float *gx, float *gcols, int B, int ych, int yh, int yw,
                                               int xch, int kh, int kw, int pad, int stride, int dilation,
                                               int xh, int xw)
{
    if (ag_status_t s = conv_dims("conv2d_transpose", B, xch, xh, xw, ych, kh, kw, pad, stride, dilation)) return s;
    AG_REQUIRE(yh >= 0 && yw >= 0, AG_ERR_INVALID_DIMS, "conv2d_transpose: negative extent (%dx%d)", yh, yw);
    const long long M = (long long)xch * kh * kw, P = (long long)yh * yw;
    AG_REQUIRE(M <= 0x7fffffff && P <= 0x7fffffff, AG_ERR_INVALID_DIMS,
               "conv2d_transpose: matrix extent overflows int");
    // every column position must map inside [-pad, x + pad): same geometry as the forward conv
    AG_REQUIRE(yh == 0 || yw == 0 ||
                   ((yh - 1) * stride + dilation * (kh - 1) + 1 <= xh + 2 * pad &&
                    (yw - 1) * stride + dilation * (kw - 1) + 1 <= xw + 2 * pad),
               AG_ERR_INCOMPATIBLE_SHAPE,
               "conv2d_transpose: output %dx%d too small for input %dx%d (k=%dx%d stride=%d pad=%d dilation=%d)", xh,
               xw, yh, yw, kh, kw, stride, pad, dilation);
    // gcols_b[M x P] = w^T[M x ych] * gy_b[ych x P]               conv2d_transpose.rs:114-116,167-182
    if (ag_status_t s = ag_gemm_f32(stream, 1, 0, (int)M, (int)P, ych, 1.f, w, (int)M, 0, gy, (int)P,
                                    (long long)ych * P, 0.f, gcols, (int)P, M * P, B))
        return s;
    return ag_col2im_f32(stream, gcols, gx, B, xch, xh, xw, kh, kw, pad, pad, stride, stride, dilation, dilation,
                         yh, yw);
}

extern "C" ag_status_t ag_conv2d_transpose_filter_grad_f32(ag_stream_t stream, const float *x,
                                                           const float *gy, float *gw, float *gycols, int B,
                                                           int ych, int yh, int yw, int xch, int H, int W,
                                                           int kh, int kw, int pad, int stride, int dilation,
                                                           void *ws, size_t ws_bytes)
{
    if (ag_status_t s = conv_dims("conv2d_transpose_filter_grad", B, xch, H, W, ych, kh, kw, pad, stride, dilation))
        return s;
    AG_REQUIRE(H + 2 * pad >= dilation * (kh - 1) + 1 && W + 2 * pad >= dilation * (kw - 1) + 1,
               AG_ERR_INCOMPATIBLE_SHAPE, "conv2d_transpose_filter_grad: filter extent exceeds the padded gradient (%dx%d)",
               H, W);
    AG_REQUIRE(ag_conv_out_size(H, kh, pad, stride, dilation) == yh &&
                   ag_conv_out_size(W, kw, pad, stride, dilation) == yw,
               AG_ERR_INCOMPATIBLE_SHAPE,
               "conv2d_transpose_filter_grad: gradient %dx%d does not reduce to the input's %dx%d", H, W, yh, yw);
    const long long N = (long long)xch * kh * kw, P = (long long)yh * yw;
    AG_REQUIRE(N <= 0x7fffffff && P <= 0x7fffffff, AG_ERR_INVALID_DIMS,
               "conv2d_transpose_filter_grad: matrix extent overflows int");
    // gy -> columns                                              conv2d_transpose.rs:331-345
    if (ag_status_t s = ag_im2col_f32(stream, gy, gycols, B, xch, H, W, kh, kw, pad, pad, stride, stride, dilation,
                                      dilation))
        return s;
    // gw[ych x N] = sum_b x_b[ych x P] * gycols_b[N x P]^T        conv2d_transpose.rs:354-381
    return ag_gemm_batchsum_f32(stream, 0, 1, ych, (int)N, (int)P, 1.f, x, (int)P, (long long)ych * P, gycols,
                                (int)P, N * P, 0.f, gw, (int)N, B, ws, ws_bytes);
}
