/*
 * ag_hip.h -- C ABI of the MI355X (gfx950) implementation of rust-autograd's
 * convolution / matmul / pooling / reduction / Adam operators.
 *
 * This is the boundary a Rust `extern "C"` block (or any other FFI) binds.  It
 * follows the convention the reference already uses for its only foreign calls,
 * `cblas_sgemm` through cblas-sys (src/tensor_ops/blas_ffi.rs:2,15; call site
 * src/tensor_ops/conv_ops/conv2d.rs:87-102): raw pointers, integer extents and
 * leading dimensions, no ownership transfer.  Additions: every pointer is a
 * DEVICE pointer to contiguous row-major f32, and every call takes a HIP stream.
 *
 * Rules that hold for every entry point
 *   - the caller owns all buffers, including workspaces (sizes come from the
 *     matching *_workspace function); the library never allocates or frees;
 *   - work is enqueued on `stream` and the call returns without synchronising;
 *   - the return value is an ag_status_t; a non-zero status leaves a
 *     human-readable message for the calling thread in ag_last_error();
 *   - status 1..5 are the five variants of the reference's `OpError`
 *     (src/op.rs:66-73) in declaration order; 100 + n is hipError_t n;
 *   - nothing throws or aborts across this boundary;
 *   - functions are re-entrant: the mutable state of the library is the
 *     thread-local error string, caches of device properties that are filled
 *     once under a lock, and the fixed scratch array of ag_matmul_f32_noalloc
 *     (see there).  The library also exports a few ag_test_* symbols for its own
 *     test-suite (rust-autograd_amd/csrc/ag_test_hooks.h); they set thread-local
 *     overrides and are not part of this boundary.
 */
#ifndef AG_HIP_H
#define AG_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Everything declared here is exported from libag_hip.so (the library itself is built with
 * hidden default visibility). */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

typedef int ag_status_t;
typedef void *ag_stream_t; /* hipStream_t */

enum {
    AG_OK = 0,
    AG_ERR_NDARRAY = 1,            /* OpError::NdArrayError      */
    AG_ERR_INCOMPATIBLE_SHAPE = 2, /* OpError::IncompatibleShape */
    AG_ERR_TYPE_UNSUPPORTED = 3,   /* OpError::TypeUnsupported   */
    AG_ERR_INVALID_DIMS = 4,       /* OpError::InvalidDims       */
    AG_ERR_OUT_OF_BOUNDS = 5,      /* OpError::OutOfBounds       */
    AG_ERR_HIP_BASE = 100          /* 100 + hipError_t           */
};

/* Message of the last non-zero status returned to the calling thread. */
const char *ag_last_error(void);

/* Library identification: "ag_hip <version> gfx950". */
const char *ag_version(void);

/* ---- geometry helpers (pure host arithmetic) ------------------------------------------------ */

/* Convolution output extent, (x + 2p - (d(k-1)+1))/s + 1.  conv_ops/mod.rs:89-90, conv2d.rs:391-392 */
int ag_conv_out_size(int x, int k, int pad, int stride, int dilation);
/* Extent Conv2DTranspose reconstructs for its output, s(y-1) - 2p + d(k-1)+1.  conv2d_transpose.rs:55-56 */
int ag_conv_transpose_out_size(int y, int k, int pad, int stride, int dilation);
/* Pooling output extent, (x + 2p - size)/s + 1.  max_pool2d.rs:183-184 */
int ag_pool_out_size(int x, int size, int pad, int stride);
/* Input extent MaxPool2DGrad reconstructs, s(y-1) - 2p + size.  max_pool2d.rs:263-264 */
int ag_pool_grad_in_size(int y, int size, int pad, int stride);

/* ---- im2col / col2im ------------------------------------------------------------------------ */

/* Replaces im2col / im2col_batch (conv_ops/mod.rs:73-124, 126-176).
 * x [B,C,H,W] -> cols [B, C*kh*kw, OH*OW], cols[b][(c,ky,kx)][(oy,ox)] =
 * x[b][c][oy*sh-ph+ky*dh][ox*sw-pw+kx*dw], zero outside the image. */
ag_status_t ag_im2col_f32(ag_stream_t stream, const float *x, float *cols, int B, int C, int H,
                          int W, int kh, int kw, int ph, int pw, int sh, int sw, int dh, int dw);

/* Replaces col2im (conv_ops/mod.rs:178-223) applied to every image, including the zero fill of
 * the destination its caller performs (conv2d_transpose.rs:152).  cols [B, C*kh*kw, OH*OW] ->
 * gx [B,C,H,W].  Contributions to one pixel are added in (ky, kx) ascending order, which is the
 * reference's order, so the result is bit-identical to it for identical cols. */
ag_status_t ag_col2im_f32(ag_stream_t stream, const float *cols, float *gx, int B, int C, int H,
                          int W, int kh, int kw, int ph, int pw, int sh, int sw, int dh, int dw,
                          int OH, int OW);

/* ---- GEMM ----------------------------------------------------------------------------------- */

/* Replaces cblas_sgemm(RowMajor, ...) as called at conv2d.rs:87-102, 246-261, 670-686,
 * conv2d_transpose.rs:167-182, 365-380 and dot_ops.rs:209-229, 352-368, extended to a strided
 * batch:  C_i = alpha * op(A_i) * op(B_i) + beta * C_i  for i in [0, batch), X_i = X + i*strideX
 * (a stride of 0 shares the operand).  trans* are 0 / 1.  Runs on fp32 MFMA. */
ag_status_t ag_gemm_f32(ag_stream_t stream, int transA, int transB, int M, int N, int K,
                        float alpha, const float *A, int lda, long long strideA, const float *B,
                        int ldb, long long strideB, float beta, float *C, int ldc,
                        long long strideC, int batch);

/* C = alpha * sum_{i<batch} op(A_i) * op(B_i) + beta*C: the image-sequential accumulation of
 * conv2d.rs:668-687 and conv2d_transpose.rs:362-381 (beta = 0 for the first image, 1 after) done
 * as one split-K launch plus a fixed-order second pass (deterministic; summation order differs
 * from the reference's, results agree to rounding).  `ws` must hold
 * ag_gemm_batchsum_f32_workspace(...) bytes. */
size_t ag_gemm_batchsum_f32_workspace(int M, int N, int K, int batch);
ag_status_t ag_gemm_batchsum_f32(ag_stream_t stream, int transA, int transB, int M, int N, int K,
                                 float alpha, const float *A, int lda, long long strideA,
                                 const float *B, int ldb, long long strideB, float beta, float *C,
                                 int ldc, int batch, void *ws, size_t ws_bytes);

/* Replaces MatMul::compute (dot_ops.rs:564-606, mat_mul_impl_blas :142-234): C[M x N] = op(A) . op(B),
 * row-major, alpha 1, beta 0.  Same result as ag_gemm_f32 with batch 1; a product with few output
 * tiles and a long contraction (K >= 512, e.g. the [128,3136].[3136,10] dense layer of
 * examples/cnn_mnist.rs) is cut into slices of K that are computed by different blocks and summed in
 * slice order, which needs the workspace. */
size_t ag_matmul_f32_workspace(int M, int N, int K);
ag_status_t ag_matmul_f32(ag_stream_t stream, int transA, int transB, int M, int N, int K,
                          const float *A, int lda, const float *B, int ldb, float *C, int ldc,
                          void *ws, size_t ws_bytes);

/* ---- convolution operators ------------------------------------------------------------------ */

/* Replaces Conv2D::compute -> conv2d_impl -> fast_im2col_gemm_fused_kernel
 * (conv2d.rs:531-554, 407-487, 25-112).  x [B,C,H,W], w [K,C,kh,kw] ->
 * y [B,K,OH,OW] (op output 0) and cols [B, C*kh*kw, OH*OW] (op output 1). */
ag_status_t ag_conv2d_fwd_f32(ag_stream_t stream, const float *x, const float *w, float *y,
                              float *cols, int B, int C, int H, int W, int K, int kh, int kw,
                              int pad, int stride, int dilation);

/* Replaces Conv2DWithCols::compute (conv2d.rs:589-597, 489-529, 215-274): the GEMM half only. */
ag_status_t ag_conv2d_with_cols_f32(ag_stream_t stream, const float *cols, const float *w, float *y,
                                    int B, int CK, int P, int K);

/* Replaces Conv2DFilterGrad::compute -> conv2d_filter_grad_impl (conv2d.rs:736-744, 631-734).
 * cols [B,CK,P], gy [B,K,P] -> gw [K,CK]. */
size_t ag_conv2d_filter_grad_f32_workspace(int B, int CK, int P, int K);
ag_status_t ag_conv2d_filter_grad_f32(ag_stream_t stream, const float *cols, const float *gy,
                                      float *gw, int B, int CK, int P, int K, void *ws,
                                      size_t ws_bytes);

/* Replaces Conv2DTranspose::compute -> conv2d_transpose_impl (conv2d_transpose.rs:249-272,
 * 89-247).  gy [B,ych,yh,yw], w [ych,xch,kh,kw] -> gx [B,xch,xh,xw].  The reference derives
 * (xh,xw) with ag_conv_transpose_out_size; here they are arguments so that a convolution's input
 * gradient can be produced at the true input size.  `gcols` is caller scratch of
 * B*xch*kh*kw*yh*yw floats (the reference's temporary `cols`, conv2d_transpose.rs:148-151). */
ag_status_t ag_conv2d_transpose_f32(ag_stream_t stream, const float *gy, const float *w, float *gx,
                                    float *gcols, int B, int ych, int yh, int yw, int xch, int kh,
                                    int kw, int pad, int stride, int dilation, int xh, int xw);

/* The two stages of the column-free input gradient that ag_conv2d_transpose_f32 runs when the
 * geometry allows it (no counterpart in the reference, which always materialises the columns):
 * `prepare` writes a zero-bordered copy of gy and the filter in tap-major order into `scratch`;
 * `gemm` accumulates gx over the filter taps in implicit GEMMs that read them -- one for stride 1;
 * for stride 2 one per parity of the pixel position, whose results (kept in `scratch`) a copy
 * kernel interleaves into gx.  Stride 1 takes any dilation (the taps are read `dilation` rows and
 * elements apart in the bordered copy); stride 2 requires dilation 1.
 * ag_conv_input_grad_scratch_floats returns the
 * scratch size in floats, or 0 when the geometry is not supported (then use
 * ag_conv2d_transpose_f32). */
size_t ag_conv_input_grad_scratch_floats(int B, int ych, int yh, int yw, int xch, int kh, int kw,
                                         int pad, int stride, int dilation, int xh, int xw);
ag_status_t ag_conv_input_grad_prepare_f32(ag_stream_t stream, const float *gy, const float *w,
                                           float *scratch, int B, int ych, int yh, int yw, int xch,
                                           int kh, int kw, int pad, int stride, int dilation, int xh,
                                           int xw);
ag_status_t ag_conv_input_grad_gemm_f32(ag_stream_t stream, float *scratch, float *gx, int B,
                                        int ych, int yh, int yw, int xch, int kh, int kw, int pad,
                                        int stride, int dilation, int xh, int xw);

/* Column-free convolution (stride 1 with any dilation, or stride 2 with dilation 1): forward and
 * filter gradient without the
 * im2col columns.  No counterpart in the reference, which always materialises them (Conv2D::compute
 * -> fast_im2col_gemm_fused_kernel, conv2d.rs:25-112; conv2d_filter_grad_impl, conv2d.rs:631-734);
 * the results are those of ag_conv2d_fwd_f32 / ag_conv2d_filter_grad_f32 within the floating-point
 * tolerance (other summation order).  The forward writes a rearranged copy of x into `xpad`
 * (ag_conv2d_nocols_scratch_floats() floats; 0 = geometry not supported: C a multiple of 32, square
 * filters, for stride 2 planes of at least 128 padded elements, ...) -- the zero-bordered input for
 * stride 1, its four phase
 * planes x'[2i+a][2j+b] for stride 2 -- and runs one implicit GEMM over the filter taps.  The filter
 * gradient contracts that copy with the zero-bordered upstream gradient that
 * ag_conv_input_grad_prepare_f32 leaves at the start of its scratch (`gypad`), summed over images
 * in splits that need the workspace; for stride 1 with any padding up to the filter's reach
 * dilation*(k-1) (K a multiple of 32; the two copies always share one row pitch, their plane
 * heights differ unless the convolution keeps the size).  The contraction runs a
 * few elements past a plane, but only over zeros of both operands (the planes are sized for that),
 * so a NaN or infinity in one channel of x reaches the gradients of that channel only; within the
 * channel it can reach filter taps that the reference's columns would not pair it with (0 * NaN at
 * a border position). */
size_t ag_conv2d_nocols_scratch_floats(int B, int C, int H, int W, int K, int kh, int kw, int pad,
                                       int stride, int dilation);
ag_status_t ag_conv2d_fwd_nocols_f32(ag_stream_t stream, const float *x, const float *w, float *y,
                                     float *xpad, int B, int C, int H, int W, int K, int kh, int kw,
                                     int pad, int stride, int dilation);
/* The two stages of ag_conv2d_fwd_nocols_f32 (rearranged copy of x and tap-major filter; the GEMM).  The size that
 * ag_conv2d_nocols_scratch_floats returns may include, behind the copy and the filter, room for the partial results
 * of a contraction that the GEMM stage slices over channel groups (products with fewer tiles than the chip has CUs):
 * that part of `xpad` is written by the GEMM stage and means nothing afterwards; the copy in front of it is what
 * the filter gradient and ag_conv2d_nocols_with_filter_f32 read.  Likewise the scratch of the input gradient. */
ag_status_t ag_conv2d_nocols_prepare_f32(ag_stream_t stream, const float *x, const float *w, float *xpad,
                                         int B, int C, int H, int W, int K, int kh, int kw, int pad,
                                         int stride, int dilation);
ag_status_t ag_conv2d_nocols_gemm_f32(ag_stream_t stream, float *xpad, float *y, int B, int C,
                                      int H, int W, int K, int kh, int kw, int pad, int stride,
                                      int dilation);
/* The forward GEMM over an existing rearranged copy with another filter: what Conv2DWithCols
 * (conv2d.rs:589-629) becomes when its "columns" input is such a copy.  wf: K*C*kh*kw floats. */
ag_status_t ag_conv2d_nocols_with_filter_f32(ag_stream_t stream, const float *xpad, const float *w,
                                             float *wf, float *y, int B, int C, int H, int W, int K,
                                             int kh, int kw, int pad, int stride, int dilation);
/* 0 = geometry not supported by the column-free filter gradient. */
size_t ag_conv2d_filter_grad_nocols_f32_workspace(int B, int C, int H, int W, int K, int kh, int kw,
                                                  int pad, int stride, int dilation);
ag_status_t ag_conv2d_filter_grad_nocols_f32(ag_stream_t stream, const float *xpad, const float *gypad,
                                             float *gw, int B, int C, int H, int W, int K, int kh,
                                             int kw, int pad, int stride, int dilation, void *ws,
                                             size_t ws_bytes);

/* Replaces Conv2DTransposeFilterGrad::compute -> conv2d_transpose_filter_grad_impl
 * (conv2d_transpose.rs:433-451, 303-431).  x [B,ych,yh,yw] (input of the transposed conv),
 * gy [B,xch,H,W] (gradient of its output) -> gw [ych,xch,kh,kw].  `gycols` is caller scratch of
 * B*xch*kh*kw*yh*yw floats; `ws` holds ag_conv2d_filter_grad_f32_workspace(B, xch*kh*kw, yh*yw, ych). */
ag_status_t ag_conv2d_transpose_filter_grad_f32(ag_stream_t stream, const float *x, const float *gy,
                                                float *gw, float *gycols, int B, int ych, int yh,
                                                int yw, int xch, int H, int W, int kh, int kw,
                                                int pad, int stride, int dilation, void *ws,
                                                size_t ws_bytes);

/* ---- max pooling ---------------------------------------------------------------------------- */

/* Replaces MaxPool2D::compute -> max_pool_f32 (max_pool2d.rs:166-227, 21-85).  x [B,C,H,W] ->
 * y, argmax [B,C,OH,OW]; argmax holds the flat offset of the first strict maximum inside the whole
 * x tensor converted to f32 by value, as the reference stores it.  `taps` (may be NULL; no
 * counterpart in the reference) receives one byte per output: dy*size + dx of that maximum inside
 * its window, 255 when no element exceeded -FLT_MAX (an all-NaN window).  It is the exact form of
 * the selection -- the f32 offset loses its low bits once x has more than 2^24 elements -- and
 * needs size <= 15.  pad must be 0: the reference's unsigned `i*stride - pad` is only defined
 * there (max_pool2d.rs:43,53). */
ag_status_t ag_maxpool2d_fwd_f32(ag_stream_t stream, const float *x, float *y, float *argmax,
                                 uint8_t *taps, int B, int C, int H, int W, int size, int pad,
                                 int stride);

/* ReLU::compute (activation_ops.rs:154-159), optionally with the AddOp in front of it (b != NULL: r = relu(a + b), b of
 * a's rank with extents bshape[i] equal to a's or 1, as for ag_add_broadcast_relu_f32), followed by MaxPool2D::compute
 * with a 2 x 2 window at stride 2 in ONE pass over even planes: the relu -> max_pool2d step of a conv block.  Writes r
 * [B,C,H,W] (the ReLU's result, which the backward reads) and y, argmax, taps [B,C,H/2,W/2] exactly as ag_relu_f32 /
 * ag_add_broadcast_relu_f32 followed by ag_maxpool2d_fwd_f32 would (same bits).  An optional fusion with no node of its
 * own in the reference: an evaluator may use it when it is about to evaluate such a pooling whose input has not been
 * computed yet.  H and W even; a and r 8-byte aligned. */
ag_status_t ag_relu_maxpool2d_2x2_f32(ag_stream_t stream, const float *a, const float *b, const int *bshape, float *r,
                                      float *y, float *argmax, uint8_t *taps, int B, int C, int H, int W);

/* Replaces MaxPool2DGrad::compute -> max_pool_grad_f32 (max_pool2d.rs:245-279, 111-135).
 * gy [B,C,OH,OW] -> gx [B,C,H,W] (zero filled, then gx[argmax[i]] += gy[i] in ascending i; done
 * here as a gather that visits the candidate windows of each pixel in that same order, so sums
 * are bit-identical).  (H,W) are explicit; the reference reconstructs them with
 * ag_pool_grad_in_size.  Uses `taps` when it is non-NULL, else the f32 argmax, which is exact
 * only while B*C*H*W <= 2^24 (AG_ERR_INVALID_DIMS beyond that). */
ag_status_t ag_maxpool2d_bwd_f32(ag_stream_t stream, const float *gy, const float *argmax,
                                 const uint8_t *taps, float *gx, int B, int C, int H, int W,
                                 int size, int pad, int stride);

/* MaxPool2DGrad::compute followed by the gradient of the ReLU in front of the pooling
 * (activation_ops.rs:161-166: greater(x, 0) * gy), in one pass over gx:
 * gx = greater(relu_x, 0) * max_pool2d_grad(gy), with the bits of the two operators run one after the
 * other.  relu_x [B,C,H,W] is the ReLU's input, or its output (same sign pattern).  The other
 * arguments are those of ag_maxpool2d_bwd_f32. */
ag_status_t ag_maxpool2d_bwd_relu_f32(ag_stream_t stream, const float *gy, const float *argmax,
                                      const uint8_t *taps, const float *relu_x, float *gx, int B,
                                      int C, int H, int W, int size, int pad, int stride);

/* Replaces MaxPool2DGradGrad::compute -> max_pool_grad_grad_f32 (max_pool2d.rs:297-331, 137-159):
 * ggy[i] = ggx[argmax[i]].  Same taps / argmax rule as the backward. */
ag_status_t ag_maxpool2d_gradgrad_f32(ag_stream_t stream, const float *ggx, const float *argmax,
                                      const uint8_t *taps, float *ggy, int B, int C, int H,
                                      int W, int size, int pad, int stride);

/* ---- reductions ----------------------------------------------------------------------------- */

/* Replaces ReduceSumToScalar::compute (reduction_ops.rs:123-128): out[0] = sum of x[0..n). */
size_t ag_sum_all_f32_workspace(size_t n);
ag_status_t ag_sum_all_f32(ag_stream_t stream, const float *x, size_t n, float *out, void *ws,
                           size_t ws_bytes);

/* Replaces ReduceSum::compute / ReduceMean::compute -> compute_reduce_sum (reduction_ops.rs:
 * 161-170, 187-215, 54-103).  x has `rank` extents `shape`; `axes` (unique, already normalised to
 * [0,rank)) are folded from the last to the first; mean != 0 multiplies by the f32 reciprocal of
 * the reduced length (reduction_ops.rs:198-209).  out receives prod(shape)/prod(reduced) values
 * (keep_dims only relabels the shape). */
size_t ag_reduce_sum_f32_workspace(const int *shape, int rank, const int *axes, int n_axes);
ag_status_t ag_reduce_sum_f32(ag_stream_t stream, const float *x, float *out, const int *shape,
                              int rank, const int *axes, int n_axes, int mean, void *ws,
                              size_t ws_bytes);

/* Replaces ReduceGradCommon::compute and ReduceSumToScalarGrad::compute (reduction_ops.rs:
 * 459-512, 141-150): broadcast gy (x's shape with the listed axes set to 1) to x's shape. */
ag_status_t ag_broadcast_grad_f32(ag_stream_t stream, const float *gy, float *gx, const int *shape,
                                  int rank, const int *axes, int n_axes);

/* ---- Adam ----------------------------------------------------------------------------------- */

/* Replaces AdamOp::compute (gradient_descent_ops/adam.rs:11-58), one fused pass, in place on
 * param, m, v; t (one float in device memory, the reference's step counter variable) is read by
 * the update and incremented afterwards on the same stream. */
ag_status_t ag_adam_update_f32(ag_stream_t stream, float *param, const float *grad, float *m,
                               float *v, float *t, size_t n, float alpha, float eps, float b1,
                               float b2);

/* The AdamOp::compute of `count` parameters (one optimizer step: Adam::compute builds one AdamOp
 * per parameter, optimizers/adam.rs:116-154) in one launch plus one for the step counters.  The
 * six tables are host arrays of `count` entries (device pointers, element counts); they are read
 * before the call returns.  Per element the arithmetic is ag_adam_update_f32's, so the results
 * equal `count` separate calls.  No two entries may share param, m, v or t
 * (AG_ERR_INVALID_DIMS); count is at most ag_adam_update_multi_max(). */
int ag_adam_update_multi_max(void);
ag_status_t ag_adam_update_multi_f32(ag_stream_t stream, int count, float *const *params,
                                     const float *const *grads, float *const *ms, float *const *vs,
                                     float *const *ts, const size_t *ns, float alpha, float eps,
                                     float b1, float b2);

/* ---- elementwise and loss glue met on either side of the operators above -------------------- */

/* ReLU::compute, x.max(0) (activation_ops.rs:154-159). */
ag_status_t ag_relu_f32(ag_stream_t stream, const float *x, float *y, size_t n);
/* ReLU::grad as one kernel: greater(x, 0) * gy (activation_ops.rs:161-166, math_ops.rs:86-179). */
ag_status_t ag_relu_grad_f32(ag_stream_t stream, const float *x, const float *gy, float *gx,
                             size_t n);
/* AddOp with a row-vector right operand: y[r][c] = x[r][c] + bias[c] (binary_ops.rs:147-166, 304-346). */
ag_status_t ag_add_bias_f32(ag_stream_t stream, const float *x, const float *bias, float *y,
                            size_t rows, size_t cols);
/* AddOp with a right operand that has the left operand's rank and extent 1 on the axes it is
 * broadcast along, e.g. a [1,C,1,1] bias on NCHW (binary_ops.rs:147-166, 304-346; the conv biases of
 * examples/cnn_mnist.rs).  bshape[i] must be shape[i] or 1; rank <= 8. */
ag_status_t ag_add_broadcast_f32(ag_stream_t stream, const float *x, const float *b, float *y,
                                 const int *shape, const int *bshape, int rank);
/* That AddOp followed by ReLU::compute (activation_ops.rs:154-159) in one pass, y = max(x + b, 0):
 * the conv-bias-activation step of examples/cnn_mnist.rs.  The sum is rounded to f32 before the
 * maximum, so the result has the bits of ag_add_broadcast_f32 followed by ag_relu_f32. */
ag_status_t ag_add_broadcast_relu_f32(ag_stream_t stream, const float *x, const float *b, float *y,
                                      const int *shape, const int *bshape, int rank);
/* MaybeReduceSum for that operand: out[c] = sum_r gy[r][c], r ascending (binary_ops.rs:39-105). */
ag_status_t ag_bias_grad_f32(ag_stream_t stream, const float *gy, float *out, size_t rows,
                             size_t cols);
/* AddN::compute (array_ops.rs:503-535): out = ((x0 + x1) + x2) + ...; xs is a HOST array of
 * `count` device pointers (count <= 8). */
ag_status_t ag_add_n_f32(ag_stream_t stream, const float *const *xs, int count, float *out,
                         size_t n);
/* Same-shape MulOp (binary_ops.rs:209-237) and scalar scaling. */
ag_status_t ag_mul_f32(ag_stream_t stream, const float *a, const float *b, float *out, size_t n);
ag_status_t ag_scale_f32(ag_stream_t stream, const float *a, float s, float *out, size_t n);
/* Division by a scalar, out = a / s: the `broadcast / reduction_len` of ReduceMean::grad
 * (reduction_ops.rs:231-234).  out may alias a. */
ag_status_t ag_div_scalar_f32(ag_stream_t stream, const float *a, float s, float *out, size_t n);
/* Fill with a constant (zeros / ones / scalar, const_gen_ops.rs:16-90). */
ag_status_t ag_fill_f32(ag_stream_t stream, float *out, float value, size_t n);
/* SparseSoftmaxCrossEntropy::compute (xent_ops.rs:63-115): logits [rows,classes], labels [rows]
 * stored as f32 -> loss [rows,1] (output 0) and log_softmax [rows,classes] (output 1).  A label that
 * is negative, not finite or >= classes makes the reference panic (xent_ops.rs:96-104); here that
 * row's loss, and its gradient row in the function below, are NaN. */
ag_status_t ag_sparse_softmax_xent_f32(ag_stream_t stream, const float *logits, const float *labels,
                                       float *loss, float *log_softmax, size_t rows,
                                       size_t classes);
/* SparseSoftmaxCrossEntropyGrad::compute (xent_ops.rs:139-153). */
ag_status_t ag_sparse_softmax_xent_grad_f32(ag_stream_t stream, const float *log_softmax,
                                            const float *labels, const float *gy, float *gx,
                                            size_t rows, size_t classes);
/* The same gradient computed from the logits (xent_ops.rs:63-115 and 139-153 in one kernel, the bits
 * of the two functions above run one after the other), for a training step that never reads the loss
 * and so need not run the forward.  gy [rows] may be NULL: every row's upstream gradient is then
 * gy_const (a mean over the batch: 1 / rows). */
ag_status_t ag_sparse_softmax_xent_grad_logits_f32(ag_stream_t stream, const float *logits,
                                                   const float *labels, const float *gy,
                                                   float gy_const, float *gx, size_t rows,
                                                   size_t classes);

/* ---- entry point that allocates nothing ----------------------------------------------------- */

/* ag_matmul_f32 without a workspace argument.  No counterpart in the reference: it is for callers
 * that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  The partial sums of a sliced contraction go to a fixed array
 * of ag_matmul_f32_static_scratch_bytes() bytes (4 MiB) that every GPU the library runs on holds
 * until the process ends; a product whose ag_matmul_f32_workspace() exceeds that is refused with
 * AG_ERR_INVALID_DIMS.  Results are bit-identical to ag_matmul_f32.  Calls that overlap on one
 * GPU (two streams, two threads) share the array and race: serialise them.  The first call on a
 * device looks up the array's address there (hipGetSymbolAddress); no call allocates or frees. */
size_t ag_matmul_f32_static_scratch_bytes(void);
ag_status_t ag_matmul_f32_noalloc(ag_stream_t stream, int transA, int transB, int M, int N, int K,
                                  const float *A, int lda, const float *B, int ldb, float *C, int ldc);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif

#ifdef __cplusplus
}
#endif
#endif /* AG_HIP_H */
