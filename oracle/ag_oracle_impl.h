/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of rust-autograd's conv / matmul /
 * pool / reduce / Adam path, written from the reference sources read as text.
 * Nothing in the shipped GPU library links or calls this file.
 *
 * This header is included twice by ag_oracle.c, once with REAL=float (SUF=f32)
 * and once with REAL=double (SUF=f64).  The f32 instance keeps the reference's
 * own loop and accumulation orders wherever those orders are fixed by the
 * reference's source; the f64 instance is the "truth" used to attribute
 * rounding differences.
 *
 * Citations are to files under the reference's src/ directory.
 */

#ifndef REAL
#error "include from ag_oracle.c"
#endif

#define ORC_CAT_(a, b) a##_##b
#define ORC_CAT(a, b) ORC_CAT_(a, b)
#define FN(name) ORC_CAT(name, SUF)

/* ------------------------------------------------------------------------ */
/* im2col for ONE image.  tensor_ops/conv_ops/mod.rs:73-124.                 */
/* cols[c][ky][kx][oy][ox] = x[c][oy*sh - ph + ky*dh][ox*sw - PH + kx*dw]    */
/* or 0 when the source lies outside the image.  The reference subtracts ph  */
/* (not pw) from the x offset (mod.rs:98); `literal_pad` keeps that quirk,   */
/* otherwise pw is used.  Every caller in the reference passes ph == pw.     */
/* ------------------------------------------------------------------------ */
static void FN(im2col_one)(const REAL *x, REAL *cols, int C, int H, int W, int kh, int kw,
                           int ph, int pw, int sh, int sw, int dh, int dw, int literal_pad)
{
    const int OH = orc_conv_out_size(H, kh, ph, sh, dh);
    const int OW = orc_conv_out_size(W, kw, pw, sw, dw);
    const int xpad = literal_pad ? ph : pw;
    REAL *out = cols;
    for (int c = 0; c < C; ++c) {
        const REAL *plane = x + (size_t)c * H * W;
        for (int ky = 0; ky < kh; ++ky) {
            for (int kx = 0; kx < kw; ++kx) {
                int iy = ky * dh - ph;
                for (int oy = 0; oy < OH; ++oy, iy += sh) {
                    if ((unsigned)iy < (unsigned)H) {
                        int ix = kx * dw - xpad;
                        for (int ox = 0; ox < OW; ++ox, ix += sw)
                            out[ox] = ((unsigned)ix < (unsigned)W) ? plane[iy * W + ix] : (REAL)0;
                    } else {
                        for (int ox = 0; ox < OW; ++ox) out[ox] = (REAL)0;
                    }
                    out += OW;
                }
            }
        }
    }
}

/* im2col over a batch.  conv_ops/mod.rs:126-176 (rayon over images there,   */
/* OpenMP over images here).                                                  */
ORC_API void FN(orc_im2col)(const REAL *x, REAL *cols, int B, int C, int H, int W, int kh,
                            int kw, int ph, int pw, int sh, int sw, int dh, int dw,
                            int literal_pad, int threads)
{
    const int OH = orc_conv_out_size(H, kh, ph, sh, dh);
    const int OW = orc_conv_out_size(W, kw, pw, sw, dw);
    const size_t xs = (size_t)C * H * W;
    const size_t cs = (size_t)C * kh * kw * OH * OW;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
    for (int b = 0; b < B; ++b)
        FN(im2col_one)(x + b * xs, cols + b * cs, C, H, W, kh, kw, ph, pw, sh, sw, dh, dw,
                       literal_pad);
}

/* ------------------------------------------------------------------------ */
/* col2im for ONE image: scatter-add into a pre-zeroed destination.          */
/* conv_ops/mod.rs:178-223.  Order of additions: c, ky, kx, oy, ox.          */
/* ------------------------------------------------------------------------ */
static void FN(col2im_one)(const REAL *cols, REAL *gx, int C, int H, int W, int kh, int kw,
                           int ph, int pw, int sh, int sw, int dh, int dw, int OH, int OW)
{
    const REAL *in = cols;
    for (int c = 0; c < C; ++c) {
        REAL *plane = gx + (size_t)c * H * W;
        for (int ky = 0; ky < kh; ++ky) {
            for (int kx = 0; kx < kw; ++kx) {
                int iy = ky * dh - ph;
                for (int oy = 0; oy < OH; ++oy, iy += sh) {
                    if ((unsigned)iy < (unsigned)H) {
                        int ix = kx * dw - pw;
                        for (int ox = 0; ox < OW; ++ox, ix += sw)
                            if ((unsigned)ix < (unsigned)W) plane[iy * W + ix] += in[ox];
                    }
                    in += OW;
                }
            }
        }
    }
}

/* col2im over a batch.  gx is [B,C,H,W]; cols is [B][C*kh*kw][OH*OW] where  */
/* OH,OW are passed explicitly (conv2d_transpose.rs derives H,W from them).  */
ORC_API void FN(orc_col2im)(const REAL *cols, REAL *gx, int B, int C, int H, int W, int kh,
                            int kw, int ph, int pw, int sh, int sw, int dh, int dw, int OH,
                            int OW, int threads)
{
    const size_t xs = (size_t)C * H * W;
    const size_t cs = (size_t)C * kh * kw * OH * OW;
    memset(gx, 0, sizeof(REAL) * xs * B);
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
    for (int b = 0; b < B; ++b)
        FN(col2im_one)(cols + b * cs, gx + b * xs, C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, OH,
                       OW);
}

/* ------------------------------------------------------------------------ */
/* Row-major GEMM  C = alpha*op(A)*op(B) + beta*C  with the cblas calling    */
/* convention the reference uses (conv2d.rs:87-102, dot_ops.rs:209-229).     */
/* Plain triple loop, k ascending, accumulation in REAL.  The reference's    */
/* arithmetic here is third-party (OpenBLAS via cblas-sys 0.1.4, or          */
/* matrixmultiply 0.3): their internal summation order is not reproduced,    */
/* so GEMM parity is to tolerance only.                                      */
/* ------------------------------------------------------------------------ */
static void FN(gemm_naive)(int ta, int tb, int m, int n, int k, REAL alpha, const REAL *A,
                           int lda, const REAL *B, int ldb, REAL beta, REAL *Cm, int ldc)
{
    for (int i = 0; i < m; ++i) {
        for (int j = 0; j < n; ++j) {
            REAL acc = (REAL)0;
            for (int p = 0; p < k; ++p) {
                const REAL a = ta ? A[(size_t)p * lda + i] : A[(size_t)i * lda + p];
                const REAL b = tb ? B[(size_t)j * ldb + p] : B[(size_t)p * ldb + j];
                acc += a * b;
            }
            REAL *dst = &Cm[(size_t)i * ldc + j];
            *dst = (beta == (REAL)0) ? alpha * acc : alpha * acc + beta * *dst;
        }
    }
}

/* Cache-blocked variant of the same arithmetic (i-k-j order): used when no  */
/* BLAS is loaded and the problem is too big for the triple loop.            */
static void FN(gemm_blocked)(int ta, int tb, int m, int n, int k, REAL alpha, const REAL *A,
                             int lda, const REAL *B, int ldb, REAL beta, REAL *Cm, int ldc)
{
    for (int i = 0; i < m; ++i) {
        REAL *crow = Cm + (size_t)i * ldc;
        if (beta == (REAL)0) for (int j = 0; j < n; ++j) crow[j] = (REAL)0;
        else if (beta != (REAL)1) for (int j = 0; j < n; ++j) crow[j] *= beta;
    }
    enum { KB = 256, JB = 1024 };
    for (int p0 = 0; p0 < k; p0 += KB) {
        const int p1 = p0 + KB < k ? p0 + KB : k;
        for (int j0 = 0; j0 < n; j0 += JB) {
            const int j1 = j0 + JB < n ? j0 + JB : n;
            for (int i = 0; i < m; ++i) {
                REAL *crow = Cm + (size_t)i * ldc;
                for (int p = p0; p < p1; ++p) {
                    const REAL a = alpha * (ta ? A[(size_t)p * lda + i] : A[(size_t)i * lda + p]);
                    if (!tb) {
                        const REAL *brow = B + (size_t)p * ldb;
                        for (int j = j0; j < j1; ++j) crow[j] += a * brow[j];
                    } else {
                        for (int j = j0; j < j1; ++j) crow[j] += a * B[(size_t)j * ldb + p];
                    }
                }
            }
        }
    }
}

ORC_API void FN(orc_gemm)(int ta, int tb, int m, int n, int k, REAL alpha, const REAL *A,
                          int lda, const REAL *B, int ldb, REAL beta, REAL *Cm, int ldc)
{
    if (FN(orc_blas_gemm)(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc)) return;
    if ((double)m * n * k <= 64.0 * 1024 * 1024)
        FN(gemm_naive)(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc);
    else
        FN(gemm_blocked)(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc);
}

/* The triple loop regardless of any loaded BLAS (tests use it as the fixed  */
/* arithmetic definition).                                                    */
ORC_API void FN(orc_gemm_naive)(int ta, int tb, int m, int n, int k, REAL alpha, const REAL *A,
                                int lda, const REAL *B, int ldb, REAL beta, REAL *Cm, int ldc)
{
    FN(gemm_naive)(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc);
}

/* ------------------------------------------------------------------------ */
/* Conv2D forward.  conv2d.rs:25-112 (per image: im2col then                 */
/* sgemm(N,N, m=ych, n=yh*yw, k=xch*kh*kw)), :407-487, :531-554.             */
/* Outputs y [B,K,OH,OW] and cols [B, C*kh*kw, OH*OW] (both are op outputs). */
/* ------------------------------------------------------------------------ */
ORC_API void FN(orc_conv2d_fwd)(const REAL *x, const REAL *w, REAL *y, REAL *cols, int B, int C,
                                int H, int W, int K, int kh, int kw, int pad, int stride,
                                int dil, int threads)
{
    const int OH = orc_conv_out_size(H, kh, pad, stride, dil);
    const int OW = orc_conv_out_size(W, kw, pad, stride, dil);
    const int CK = C * kh * kw, P = OH * OW;
    const size_t xs = (size_t)C * H * W, cs = (size_t)CK * P, ys = (size_t)K * P;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
    for (int b = 0; b < B; ++b) {
        FN(im2col_one)(x + b * xs, cols + b * cs, C, H, W, kh, kw, pad, pad, stride, stride, dil,
                       dil, 1);
        FN(orc_gemm)(0, 0, K, P, CK, (REAL)1, w, CK, cols + b * cs, P, (REAL)0, y + b * ys, P);
    }
}

/* Conv2DWithCols forward (GEMM only).  conv2d.rs:215-274, :489-529.         */
ORC_API void FN(orc_conv2d_with_cols)(const REAL *cols, const REAL *w, REAL *y, int B, int CK,
                                      int P, int K, int threads)
{
    const size_t cs = (size_t)CK * P, ys = (size_t)K * P;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
    for (int b = 0; b < B; ++b)
        FN(orc_gemm)(0, 0, K, P, CK, (REAL)1, w, CK, cols + b * cs, P, (REAL)0, y + b * ys, P);
}

/* Conv2DFilterGrad.  conv2d.rs:631-734: image-sequential                    */
/* sgemm(N,T, m=ych, n=kh*kw*xch, k=yh*yw, beta = 0 for image 0 else 1).     */
ORC_API void FN(orc_conv2d_filter_grad)(const REAL *cols, const REAL *gy, REAL *gw, int B,
                                        int CK, int P, int K)
{
    const size_t cs = (size_t)CK * P, gs = (size_t)K * P;
    for (int b = 0; b < B; ++b)
        FN(orc_gemm)(0, 1, K, CK, P, (REAL)1, gy + b * gs, P, cols + b * cs, P,
                     b == 0 ? (REAL)0 : (REAL)1, gw, CK);
}

/* Conv2DTranspose (conv input gradient and the public transposed conv).     */
/* conv2d_transpose.rs:89-247: per image sgemm(T,N, m=kh*kw*xch, n=yh*yw,    */
/* k=ych, lda=m) into a temporary cols buffer, then col2im.  The reference   */
/* derives the output size as s*(yh-1) - 2p + d*(kh-1) + 1 (:55-56); here it */
/* is an argument so that both that value and the true input size can be     */
/* exercised.  `gcols` (scratch, [B, C*kh*kw, yh*yw]) is returned too.       */
ORC_API void FN(orc_conv2d_transpose)(const REAL *gy, const REAL *w, REAL *gx, REAL *gcols,
                                      int B, int ych, int yh, int yw, int xch, int kh, int kw,
                                      int pad, int stride, int dil, int xh, int xw, int threads)
{
    const int M = xch * kh * kw, P = yh * yw;
    const size_t gs = (size_t)ych * P, cs = (size_t)M * P, xs = (size_t)xch * xh * xw;
    memset(gx, 0, sizeof(REAL) * xs * B);
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
    for (int b = 0; b < B; ++b) {
        FN(orc_gemm)(1, 0, M, P, ych, (REAL)1, w, M, gy + b * gs, P, (REAL)0, gcols + b * cs, P);
        FN(col2im_one)(gcols + b * cs, gx + b * xs, xch, xh, xw, kh, kw, pad, pad, stride,
                       stride, dil, dil, yh, yw);
    }
}

/* Conv2DTransposeFilterGrad.  conv2d_transpose.rs:303-431: im2col_batch on  */
/* gy (the gradient of the transposed conv's OUTPUT, [B,xch,H,W]), then the  */
/* image-sequential sgemm(N,T, m=ych, n=kh*kw*xch, k=yh*yw) with x           */
/* ([B,ych,yh,yw]) as the left operand.  `gycols` is scratch                 */
/* [B, xch*kh*kw, yh*yw].                                                    */
ORC_API void FN(orc_conv2d_transpose_filter_grad)(const REAL *x, const REAL *gy, REAL *gw,
                                                  REAL *gycols, int B, int ych, int yh, int yw,
                                                  int xch, int H, int W, int kh, int kw,
                                                  int pad, int stride, int dil, int threads)
{
    const int N = xch * kh * kw, P = yh * yw;
    FN(orc_im2col)(gy, gycols, B, xch, H, W, kh, kw, pad, pad, stride, stride, dil, dil, 1,
                   threads);
    const size_t xs = (size_t)ych * P, cs = (size_t)N * P;
    for (int b = 0; b < B; ++b)
        FN(orc_gemm)(0, 1, ych, N, P, (REAL)1, x + b * xs, P, gycols + b * cs, P,
                     b == 0 ? (REAL)0 : (REAL)1, gw, N);
}

/* ------------------------------------------------------------------------ */
/* MatMul / BatchMatMul.  dot_ops.rs:564-606, :631-695: transposes are       */
/* stride swaps of row-major operands, output row-major values.              */
/* ------------------------------------------------------------------------ */
ORC_API void FN(orc_matmul)(const REAL *a, const REAL *b, REAL *c, int m, int n, int k, int ta,
                            int tb)
{
    FN(orc_gemm)(ta, tb, m, n, k, (REAL)1, a, ta ? m : k, b, tb ? k : n, (REAL)0, c, n);
}

ORC_API void FN(orc_batch_matmul)(const REAL *a, const REAL *b, REAL *c, int batch, int m,
                                  int n, int k, int ta, int tb, int threads)
{
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
    for (int i = 0; i < batch; ++i)
        FN(orc_gemm)(ta, tb, m, n, k, (REAL)1, a + (size_t)i * m * k, ta ? m : k,
                     b + (size_t)i * k * n, tb ? k : n, (REAL)0, c + (size_t)i * m * n, n);
}

/* ------------------------------------------------------------------------ */
/* MaxPool2D forward.  conv_ops/max_pool2d.rs:21-85.  Window rows            */
/* [oy*s, min(oy*s+size, H)), same for columns, row-major scan, first strict */
/* maximum wins (`val > max`, :66), start value the most negative finite     */
/* REAL with index 0 (:51-52).  The index is the flat offset into the whole  */
/* [B,C,H,W] tensor and is stored converted to REAL by value (:74-75).       */
/* `idx_local` (may be NULL) additionally receives the exact offset inside   */
/* the (b,c) plane as int32.  pad must be 0: the reference computes          */
/* `i*stride - pad` in unsigned arithmetic (:43,53), which is only defined   */
/* for pad == 0.  Returns 0, or -1 for pad != 0.                             */
/* ------------------------------------------------------------------------ */
ORC_API int FN(orc_maxpool2d_fwd)(const REAL *x, REAL *y, REAL *argmax, int32_t *idx_local,
                                  int B, int C, int H, int W, int size, int pad, int stride)
{
    if (pad != 0) return -1;
    const int OH = (H + 2 * pad - size) / stride + 1;
    const int OW = (W + 2 * pad - size) / stride + 1;
    for (int b = 0; b < B; ++b)
        for (int c = 0; c < C; ++c) {
            const size_t plane = ((size_t)b * C + c) * H * W;
            const size_t oplane = ((size_t)b * C + c) * OH * OW;
            for (int oy = 0; oy < OH; ++oy) {
                const int h0 = oy * stride;
                const int h1 = h0 + size > H ? H : h0 + size;
                for (int ox = 0; ox < OW; ++ox) {
                    const int w0 = ox * stride;
                    const int w1 = w0 + size > W ? W : w0 + size;
                    REAL best = -REAL_MAX;
                    size_t best_i = 0;
                    int found = 0; /* did any element exceed the initial maximum? (none does in an all-NaN window) */
                    for (int h = h0; h < h1; ++h)
                        for (int ww = w0; ww < w1; ++ww) {
                            const size_t i = plane + (size_t)h * W + ww;
                            const REAL v = x[i];
                            if (v > best) { best = v; best_i = i; found = 1; }
                        }
                    const size_t o = oplane + (size_t)oy * OW + ox;
                    y[o] = best;
                    argmax[o] = (REAL)best_i;
                    if (idx_local) idx_local[o] = found ? (int32_t)(best_i - plane) : -1;
                }
            }
        }
    return 0;
}

/* MaxPool2DGrad.  max_pool2d.rs:111-135: zero gx, then in ascending output  */
/* order gx[(isize)argmax[i]] += gy[i].  gx has n_x elements (the reference  */
/* sizes it from s*(yh-1)-2p+size, :263-264; passing the true input size     */
/* keeps every index in bounds).  Returns the number of indices that fell    */
/* outside [0, n_x) and were skipped (undefined behaviour in the reference). */
ORC_API long FN(orc_maxpool2d_bwd)(const REAL *gy, const REAL *argmax, REAL *gx, size_t n_y,
                                   size_t n_x)
{
    long skipped = 0;
    memset(gx, 0, sizeof(REAL) * n_x);
    for (size_t i = 0; i < n_y; ++i) {
        const long long at = (long long)argmax[i];
        if (at < 0 || (size_t)at >= n_x) { ++skipped; continue; }
        gx[at] += gy[i];
    }
    return skipped;
}

/* Same scatter driven by the exact plane-local int32 indices.               */
ORC_API void FN(orc_maxpool2d_bwd_local)(const REAL *gy, const int32_t *idx_local, REAL *gx,
                                         size_t planes, size_t plane_y, size_t plane_x)
{
    memset(gx, 0, sizeof(REAL) * planes * plane_x);
    for (size_t p = 0; p < planes; ++p)
        for (size_t i = 0; i < plane_y; ++i) {
            const int32_t at = idx_local[p * plane_y + i];
            if (at >= 0) gx[p * plane_x + at] += gy[p * plane_y + i];
            else gx[0] += gy[p * plane_y + i]; /* no element beat the start value: index 0 */
        }
}

/* MaxPool2DGradGrad.  max_pool2d.rs:137-159: ggy[i] = ggx[(isize)argmax[i]] */
ORC_API void FN(orc_maxpool2d_gradgrad)(const REAL *ggx, const REAL *argmax, REAL *ggy,
                                        size_t n_y, size_t n_x)
{
    for (size_t i = 0; i < n_y; ++i) {
        const long long at = (long long)argmax[i];
        ggy[i] = (at >= 0 && (size_t)at < n_x) ? ggx[at] : (REAL)0;
    }
}

/* ------------------------------------------------------------------------ */
/* Reductions.  reduction_ops.rs.                                            */
/* ------------------------------------------------------------------------ */

/* ReduceSumToScalar (:123-128) = ndarray's ArrayBase::sum() on a contiguous */
/* array.  That routine is third-party (ndarray 0.16, src/numeric_util.rs    */
/* `unrolled_fold`): eight running partial sums over blocks of eight, folded */
/* as acc += (p0+p4); acc += (p1+p5); acc += (p2+p6); acc += (p3+p7); then   */
/* the tail of fewer than eight elements is added in order.  Restated from   */
/* its published source; parity is to tolerance only.                        */
ORC_API REAL FN(orc_sum_all)(const REAL *x, size_t n)
{
    REAL p[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    size_t i = 0;
    for (; i + 8 <= n; i += 8)
        for (int j = 0; j < 8; ++j) p[j] = p[j] + x[i + j];
    REAL acc = (REAL)0;
    acc = acc + (p[0] + p[4]);
    acc = acc + (p[1] + p[5]);
    acc = acc + (p[2] + p[6]);
    acc = acc + (p[3] + p[7]);
    for (; i < n; ++i) acc = acc + x[i];
    return acc;
}

/* One fold_axis step (:74-89): x viewed as [outer][len][inner] -> out       */
/* [outer][inner], sequential 0 + x0 + x1 + ... along the folded axis.       */
ORC_API void FN(orc_fold_axis_sum)(const REAL *x, REAL *out, size_t outer, size_t len,
                                   size_t inner)
{
    for (size_t o = 0; o < outer; ++o)
        for (size_t i = 0; i < inner; ++i) {
            REAL acc = (REAL)0;
            for (size_t r = 0; r < len; ++r) acc = acc + x[(o * len + r) * inner + i];
            out[o * inner + i] = acc;
        }
}

/* ReduceSum (:161-170, :54-103): axes sorted ascending and folded from the  */
/* last one to the first; keep_dims only changes the shape label.  `axes`    */
/* must be unique and in range.  `mean` != 0 gives ReduceMean (:187-215):    */
/* the reduced length is accumulated as f32 and applied as a multiplication  */
/* by its reciprocal (:198-209).  out holds prod(shape)/prod(reduced) values.*/
ORC_API void FN(orc_reduce_sum)(const REAL *x, REAL *out, const int *shape, int rank,
                                const int *axes, int n_axes, int mean)
{
    int dims[16], ax[16];
    size_t total = 1;
    for (int i = 0; i < rank; ++i) { dims[i] = shape[i]; total *= (size_t)shape[i]; }
    for (int i = 0; i < n_axes; ++i) ax[i] = axes[i];
    for (int i = 1; i < n_axes; ++i)           /* insertion sort, ascending */
        for (int j = i; j > 0 && ax[j - 1] > ax[j]; --j) { int t = ax[j]; ax[j] = ax[j - 1]; ax[j - 1] = t; }
    float red_len = 1.f;
    for (int i = 0; i < n_axes; ++i) red_len *= (float)shape[ax[i]];
    REAL *cur = (REAL *)malloc(sizeof(REAL) * (total ? total : 1));
    REAL *nxt = (REAL *)malloc(sizeof(REAL) * (total ? total : 1));
    memcpy(cur, x, sizeof(REAL) * total);
    size_t cur_n = total;
    for (int a = n_axes - 1; a >= 0; --a) {
        size_t outer = 1, inner = 1;
        for (int i = 0; i < ax[a]; ++i) outer *= (size_t)dims[i];
        for (int i = ax[a] + 1; i < rank; ++i) inner *= (size_t)dims[i];
        FN(orc_fold_axis_sum)(cur, nxt, outer, (size_t)dims[ax[a]], inner);
        dims[ax[a]] = 1;
        cur_n = outer * inner;
        REAL *t = cur; cur = nxt; nxt = t;
    }
    if (mean && n_axes > 0) {
        const REAL inv = (REAL)1 / (REAL)red_len;
        for (size_t i = 0; i < cur_n; ++i) cur[i] = cur[i] * inv;
    }
    memcpy(out, cur, sizeof(REAL) * cur_n);
    free(cur);
    free(nxt);
}

/* ReduceGradCommon (:459-512) / ReduceSumToScalarGrad (:141-150): broadcast */
/* gy (shape = x's shape with the reduced axes set to 1) back to x's shape.  */
ORC_API void FN(orc_broadcast_grad)(const REAL *gy, REAL *gx, const int *shape, int rank,
                                    const int *axes, int n_axes)
{
    int reduced[16] = {0};
    size_t total = 1;
    for (int i = 0; i < n_axes; ++i) reduced[axes[i]] = 1;
    for (int i = 0; i < rank; ++i) total *= (size_t)shape[i];
    for (size_t flat = 0; flat < total; ++flat) {
        size_t rem = flat, src = 0, mul = 1;
        for (int d = rank - 1; d >= 0; --d) {
            const size_t c = rem % (size_t)shape[d];
            rem /= (size_t)shape[d];
            if (!reduced[d]) { src += c * mul; mul *= (size_t)shape[d]; }
        }
        gx[flat] = gy[src];
    }
}

/* ------------------------------------------------------------------------ */
/* AdamOp::compute.  gradient_descent_ops/adam.rs:11-58, literal operation   */
/* order: m = m*b1 + (1-b1)*g; v = v*b2 + ((1-b2)*g)*g;                       */
/* v_hat = v * (1/(1-b2^t)); m_hat = m * (1/(1-b1^t));                        */
/* m_hat /= sqrt(v_hat) + eps; p -= alpha*m_hat; t += 1.                      */
/* ------------------------------------------------------------------------ */
ORC_API void FN(orc_adam)(REAL *p, const REAL *g, REAL *m, REAL *v, REAL *t, size_t n,
                          REAL alpha, REAL eps, REAL b1, REAL b2)
{
    const REAL one = (REAL)1;
    const REAL c1 = one - b1, c2 = one - b2;
    const REAL tv = *t;
    const REAL rv = one / (one - REAL_POW(b2, tv));
    const REAL rm = one / (one - REAL_POW(b1, tv));
    for (size_t i = 0; i < n; ++i) {
        const REAL gi = g[i];
        const REAL mi = m[i] * b1 + c1 * gi;
        const REAL vi = v[i] * b2 + c2 * gi * gi;
        m[i] = mi;
        v[i] = vi;
        const REAL vh = vi * rv;
        REAL mh = mi * rm;
        mh = mh / (REAL_SQRT(vh) + eps);
        p[i] = p[i] - alpha * mh;
    }
    *t = tv + one;
}

/* ------------------------------------------------------------------------ */
/* Elementwise / loss glue met by the configurations.                        */
/* ------------------------------------------------------------------------ */

/* ReLU forward x.max(0) (activation_ops.rs:155-159) and its gradient        */
/* greater(x,0)*gy (:161-166, math_ops.rs:86-179: 1.0 where x > 0 else 0.0). */
ORC_API void FN(orc_relu)(const REAL *x, REAL *y, size_t n)
{
    for (size_t i = 0; i < n; ++i) y[i] = x[i] > (REAL)0 ? x[i] : (REAL)0;
}
ORC_API void FN(orc_relu_grad)(const REAL *x, const REAL *gy, REAL *gx, size_t n)
{
    for (size_t i = 0; i < n; ++i) gx[i] = (x[i] > (REAL)0 ? (REAL)1 : (REAL)0) * gy[i];
}

/* AddOp with a [1,cols] (or [cols]) right operand broadcast over rows       */
/* (binary_ops.rs:147-166, :304-346) and the gradient w.r.t. that operand:   */
/* MaybeReduceSum = sum over axis 0, sequential (binary_ops.rs:39-105).      */
ORC_API void FN(orc_add_bias)(const REAL *x, const REAL *bias, REAL *y, size_t rows, size_t cols)
{
    for (size_t r = 0; r < rows; ++r)
        for (size_t c = 0; c < cols; ++c) y[r * cols + c] = x[r * cols + c] + bias[c];
}

/* AddN (array_ops.rs:503-535): out = ((x0 + x1) + x2) + ...                 */
ORC_API void FN(orc_add_n)(const REAL *const *xs, int count, REAL *out, size_t n)
{
    for (size_t i = 0; i < n; ++i) {
        REAL acc = xs[0][i];
        for (int j = 1; j < count; ++j) acc = acc + xs[j][i];
        out[i] = acc;
    }
}

/* SparseSoftmaxCrossEntropy (xent_ops.rs:63-137) on logits [rows, classes], */
/* labels stored as REAL: log_softmax = x - logsumexp(x) with the max trick  */
/* of math_ops.rs:540-593 (max, sum of exp(x-max), ln, + max), loss[r] =     */
/* -log_softmax[r][label]; outputs loss [rows,1] and log_softmax.            */
ORC_API void FN(orc_sparse_softmax_xent)(const REAL *logits, const REAL *labels, REAL *loss,
                                         REAL *log_softmax, size_t rows, size_t classes)
{
    for (size_t r = 0; r < rows; ++r) {
        const REAL *row = logits + r * classes;
        REAL mx = row[0];
        for (size_t c = 1; c < classes; ++c) mx = row[c] > mx ? row[c] : mx;
        REAL s = (REAL)0;
        for (size_t c = 0; c < classes; ++c) s = s + REAL_EXP(row[c] - mx);
        const REAL lse = REAL_LOG(s) + mx;
        for (size_t c = 0; c < classes; ++c) log_softmax[r * classes + c] = row[c] - lse;
        loss[r] = -log_softmax[r * classes + (size_t)labels[r]];
    }
}

/* SparseSoftmaxCrossEntropyGrad (xent_ops.rs:139-158): softmax = exp(log    */
/* softmax); subtract 1 at the label; multiply by gy [rows,1].               */
ORC_API void FN(orc_sparse_softmax_xent_grad)(const REAL *log_softmax, const REAL *labels,
                                              const REAL *gy, REAL *gx, size_t rows,
                                              size_t classes)
{
    for (size_t r = 0; r < rows; ++r)
        for (size_t c = 0; c < classes; ++c) {
            REAL s = REAL_EXP(log_softmax[r * classes + c]);
            if (c == (size_t)labels[r]) s = s - (REAL)1;
            gx[r * classes + c] = s * gy[r];
        }
}

#undef FN
#undef ORC_CAT
#undef ORC_CAT_
