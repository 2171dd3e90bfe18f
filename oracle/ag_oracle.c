/*
 * TEST INFRASTRUCTURE ONLY.
 *
 * CPU oracle for the conv / matmul / pool / reduce / Adam path of
 * rust-autograd, restated from the reference's Rust sources (read as text;
 * the reference itself needs cargo + crates.io and cannot be built here).
 * It exists to check the GPU library and to be timed as the CPU baseline.
 * The GPU library never links, loads or calls anything in this directory.
 *
 * What pins each function (see tests/test_oracle_*.py):
 *   im2col            reference known-answer vector conv_ops/mod.rs:26-71,
 *                     brute-force index definition, adjoint identity
 *   col2im / conv2d_transpose
 *                     reference vector conv2d_transpose.rs:482-509, adjoint
 *                     identity <im2col(x),c> == <x,col2im(c)>, torch CPU
 *                     conv_transpose2d
 *   conv2d fwd / filter grad / transpose filter grad
 *                     direct 7-loop convolution and torch CPU autograd in f64
 *   gemm / matmul / batch_matmul
 *                     reference integer vectors tests/test_tensor_ops_eval.rs
 *                     :71-185, numpy f64 matmul
 *   maxpool fwd/bwd/gradgrad
 *                     reference vector max_pool2d.rs:90-109, brute force,
 *                     tie / NaN / clipped-window cases
 *   sum_all / reduce_sum / reduce_mean / broadcast_grad
 *                     reference value tests/test_tensor_ops_eval.rs:48-56,
 *                     closed forms, numpy f64
 *   adam              closed form of the first step, f64 recurrence
 *   relu / add_bias / add_n / sparse_softmax_xent(+grad)
 *                     numpy / scipy.special.logsumexp definitions
 *
 * Third-party arithmetic that is NOT under the reference tree and is
 * therefore matched to tolerance only: SGEMM (cblas-sys 0.1.4 -> OpenBLAS, or
 * matrixmultiply 0.3) and ndarray 0.16 `sum()` / `fold_axis`.
 */

#include <dlfcn.h>
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* Output extent of a convolution axis (conv_ops/mod.rs:89-90, conv2d.rs:391-392). */
ORC_API int orc_conv_out_size(int x, int k, int p, int s, int d)
{
    return (x + 2 * p - (d * (k - 1) + 1)) / s + 1;
}

/* Output extent reconstructed by Conv2DTranspose (conv2d_transpose.rs:55-56). */
ORC_API int orc_conv_transpose_out_size(int y, int k, int p, int s, int d)
{
    return s * (y - 1) - 2 * p + (d * (k - 1) + 1);
}

/* Input extent reconstructed by MaxPool2DGrad (max_pool2d.rs:263-264). */
ORC_API int orc_pool_grad_in_size(int y, int size, int p, int s)
{
    return s * (y - 1) - 2 * p + size;
}

/* ------------------------------------------------------------------------ */
/* Optional CBLAS found at run time (the reference's `blas,openblas`        */
/* feature).  Accepts plain `cblas_sgemm` or SciPy's bundled OpenBLAS whose  */
/* LP64 symbols carry a `scipy_` prefix.                                     */
/* ------------------------------------------------------------------------ */
typedef void (*sgemm_fn)(int, int, int, int, int, int, float, const float *, int, const float *,
                         int, float, float *, int);
typedef void (*dgemm_fn)(int, int, int, int, int, int, double, const double *, int,
                         const double *, int, double, double *, int);
typedef void (*set_threads_fn)(int);

static void *g_blas_handle = NULL;
static sgemm_fn g_sgemm = NULL;
static dgemm_fn g_dgemm = NULL;
static set_threads_fn g_set_threads = NULL;
static char g_blas_name[512] = "none (built-in loops, not OpenBLAS)";

ORC_API int orc_blas_load(const char *path)
{
    void *h = dlopen(path, RTLD_NOW | RTLD_LOCAL);
    if (!h) return 0;
    sgemm_fn s = (sgemm_fn)dlsym(h, "cblas_sgemm");
    dgemm_fn d = (dgemm_fn)dlsym(h, "cblas_dgemm");
    set_threads_fn t = (set_threads_fn)dlsym(h, "openblas_set_num_threads");
    if (!s) {
        s = (sgemm_fn)dlsym(h, "scipy_cblas_sgemm");
        d = (dgemm_fn)dlsym(h, "scipy_cblas_dgemm");
        t = (set_threads_fn)dlsym(h, "scipy_openblas_set_num_threads");
    }
    if (!s || !d) { dlclose(h); return 0; }
    g_blas_handle = h;
    g_sgemm = s;
    g_dgemm = d;
    g_set_threads = t;
    snprintf(g_blas_name, sizeof g_blas_name, "%s", path);
    return 1;
}

ORC_API void orc_blas_unload(void)
{
    g_sgemm = NULL;
    g_dgemm = NULL;
    g_set_threads = NULL;
    snprintf(g_blas_name, sizeof g_blas_name, "none (built-in loops, not OpenBLAS)");
}

ORC_API const char *orc_blas_name(void) { return g_blas_name; }

ORC_API void orc_blas_set_threads(int n)
{
    if (g_set_threads) g_set_threads(n);
}

enum { CblasRowMajor = 101, CblasNoTrans = 111, CblasTrans = 112 };

static int orc_blas_gemm_f32(int ta, int tb, int m, int n, int k, float alpha, const float *A,
                             int lda, const float *B, int ldb, float beta, float *C, int ldc)
{
    if (!g_sgemm) return 0;
    g_sgemm(CblasRowMajor, ta ? CblasTrans : CblasNoTrans, tb ? CblasTrans : CblasNoTrans, m, n,
            k, alpha, A, lda, B, ldb, beta, C, ldc);
    return 1;
}

static int orc_blas_gemm_f64(int ta, int tb, int m, int n, int k, double alpha, const double *A,
                             int lda, const double *B, int ldb, double beta, double *C, int ldc)
{
    if (!g_dgemm) return 0;
    g_dgemm(CblasRowMajor, ta ? CblasTrans : CblasNoTrans, tb ? CblasTrans : CblasNoTrans, m, n,
            k, alpha, A, lda, B, ldb, beta, C, ldc);
    return 1;
}

#define REAL float
#define SUF f32
#define REAL_MAX FLT_MAX
#define REAL_POW powf
#define REAL_SQRT sqrtf
#define REAL_EXP expf
#define REAL_LOG logf
#include "ag_oracle_impl.h"
#undef REAL
#undef SUF
#undef REAL_MAX
#undef REAL_POW
#undef REAL_SQRT
#undef REAL_EXP
#undef REAL_LOG

#define REAL double
#define SUF f64
#define REAL_MAX DBL_MAX
#define REAL_POW pow
#define REAL_SQRT sqrt
#define REAL_EXP exp
#define REAL_LOG log
#include "ag_oracle_impl.h"
#undef REAL
#undef SUF
#undef REAL_MAX
#undef REAL_POW
#undef REAL_SQRT
#undef REAL_EXP
#undef REAL_LOG
