// Elementwise and loss glue that sits on either side of the conv / matmul / pool operators in the
// reference's graphs: ReLU and its gradient, bias add and its column-sum gradient, AddN, Mul,
// fills, and sparse softmax cross-entropy.  All HBM-bound single-pass kernels.
#include <cfloat>

#include "ag_internal.h"

namespace ag {

static unsigned ew_grid(size_t n, int per_thread)
{
    size_t b = (n + 256ull * per_thread - 1) / (256ull * per_thread);
    if (b < 1) b = 1;
    if (b > 131072) b = 131072;
    return (unsigned)b;
}

#define AG_EW_LOOP(i, n) \
    for (size_t i = blockIdx.x * 256ull + threadIdx.x; i < (n); i += gridDim.x * 256ull)

// activation_ops.rs:155-159  x.max(0)  (f32::max: NaN input yields 0)
__global__ __launch_bounds__(256) void relu_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                   size_t n)
{
    AG_EW_LOOP(i, n) { const float v = x[i]; y[i] = v > 0.f ? v : 0.f; }
}

// activation_ops.rs:161-166  greater(x, 0) * gy
__global__ __launch_bounds__(256) void relu_grad_kernel(const float *__restrict__ x,
                                                        const float *__restrict__ gy,
                                                        float *__restrict__ gx, size_t n)
{
    AG_EW_LOOP(i, n) gx[i] = (x[i] > 0.f ? 1.f : 0.f) * gy[i];
}

__global__ __launch_bounds__(256) void add_bias_kernel(const float *__restrict__ x,
                                                       const float *__restrict__ bias,
                                                       float *__restrict__ y, size_t n, size_t cols)
{
    AG_EW_LOOP(i, n) y[i] = x[i] + bias[i % cols];
}

// Right operand broadcast along any of its axes of extent 1.  `dims` are the left operand's extents
// after adjacent axes with the same broadcast state have been merged (outermost first), `bstride`
// the right operand's element stride for each merged axis (0 where it is broadcast).
struct BroadcastGeom {
    unsigned dims[6];
    unsigned bstride[6];
    int rank;
};

__global__ __launch_bounds__(256) void add_broadcast_kernel(const float *__restrict__ x,
                                                            const float *__restrict__ b,
                                                            float *__restrict__ y, size_t n, BroadcastGeom g)
{
    AG_EW_LOOP(i, n)
    {
        size_t rest = i, bi = 0;
        for (int d = g.rank - 1; d > 0; --d) {
            const size_t q = rest / g.dims[d];
            bi += (rest - q * g.dims[d]) * g.bstride[d];
            rest = q;
        }
        bi += rest * g.bstride[0];
        y[i] = x[i] + b[bi];
    }
}

// out[c] = sum over rows, ascending (ndarray sum_axis(0) order used by MaybeReduceSum).
__global__ __launch_bounds__(256) void bias_grad_kernel(const float *__restrict__ gy,
                                                        float *__restrict__ out, size_t rows, size_t cols)
{
    AG_EW_LOOP(c, cols)
    {
        float acc = 0.f;
        for (size_t r = 0; r < rows; ++r) acc += gy[r * cols + c];
        out[c] = acc;
    }
}

struct PtrPack {
    const float *p[8];
};

__global__ __launch_bounds__(256) void add_n_kernel(PtrPack xs, int count, float *__restrict__ out, size_t n)
{
    AG_EW_LOOP(i, n)
    {
        float acc = xs.p[0][i];
        for (int j = 1; j < count; ++j) acc += xs.p[j][i];
        out[i] = acc;
    }
}

__global__ __launch_bounds__(256) void mul_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                  float *__restrict__ out, size_t n)
{
    AG_EW_LOOP(i, n) out[i] = a[i] * b[i];
}

__global__ __launch_bounds__(256) void scale_kernel(const float *__restrict__ a, float s,
                                                    float *__restrict__ out, size_t n)
{
    AG_EW_LOOP(i, n) out[i] = a[i] * s;
}

__global__ __launch_bounds__(256) void div_scalar_kernel(const float *__restrict__ a, float s,
                                                         float *__restrict__ out, size_t n)
{
    AG_EW_LOOP(i, n) out[i] = a[i] / s;
}

__global__ __launch_bounds__(256) void fill_kernel(float *__restrict__ out, float v, size_t n)
{
    AG_EW_LOOP(i, n) out[i] = v;
}

// One thread per row (class counts are small): log_softmax = x - (ln(sum exp(x - max)) + max),
// loss = -log_softmax[label].  xent_ops.rs:63-115, math_ops.rs:540-593.
__global__ __launch_bounds__(256) void sparse_xent_kernel(const float *__restrict__ logits,
                                                          const float *__restrict__ labels,
                                                          float *__restrict__ loss,
                                                          float *__restrict__ lsm, size_t rows,
                                                          size_t classes)
{
    AG_EW_LOOP(r, rows)
    {
        const float *row = logits + r * classes;
        float mx = -FLT_MAX;
        for (size_t c = 0; c < classes; ++c) mx = fmaxf(mx, row[c]);
        float s = 0.f;
        for (size_t c = 0; c < classes; ++c) s += expf(row[c] - mx);
        const float lse = logf(s) + mx;
        const size_t label = (size_t)labels[r];
        float picked = 0.f;
        for (size_t c = 0; c < classes; ++c) {
            const float v = row[c] - lse;
            lsm[r * classes + c] = v;
            if (c == label) picked = v;
        }
        loss[r] = -picked;
    }
}

// xent_ops.rs:139-153  (exp(log_softmax) - onehot(label)) * gy[row]
__global__ __launch_bounds__(256) void sparse_xent_grad_kernel(const float *__restrict__ lsm,
                                                               const float *__restrict__ labels,
                                                               const float *__restrict__ gy,
                                                               float *__restrict__ gx, size_t rows,
                                                               size_t classes)
{
    const size_t n = rows * classes;
    AG_EW_LOOP(i, n)
    {
        const size_t r = i / classes, c = i - r * classes;
        float s = expf(lsm[i]);
        if (c == (size_t)labels[r]) s -= 1.f;
        gx[i] = s * gy[r];
    }
}

}  // namespace ag

using namespace ag;

#define AG_EW_ENTRY(name, kernel, nexpr, ...)                                                     \
    do {                                                                                          \
        const size_t n__ = (nexpr);                                                               \
        if (n__ == 0) return AG_OK;                                                               \
        hipLaunchKernelGGL(kernel, dim3(ew_grid(n__, 4)), dim3(256), 0, as_stream(stream), __VA_ARGS__); \
        return check_launch(name);                                                                \
    } while (0)

extern "C" ag_status_t ag_relu_f32(ag_stream_t stream, const float *x, float *y, size_t n)
{
    AG_REQUIRE(n == 0 || (x && y), AG_ERR_INVALID_DIMS, "relu: null pointer");
    AG_EW_ENTRY("relu", relu_kernel, n, x, y, n);
}

extern "C" ag_status_t ag_relu_grad_f32(ag_stream_t stream, const float *x, const float *gy, float *gx,
                                        size_t n)
{
    AG_REQUIRE(n == 0 || (x && gy && gx), AG_ERR_INVALID_DIMS, "relu_grad: null pointer");
    AG_EW_ENTRY("relu_grad", relu_grad_kernel, n, x, gy, gx, n);
}

extern "C" ag_status_t ag_add_bias_f32(ag_stream_t stream, const float *x, const float *bias, float *y,
                                       size_t rows, size_t cols)
{
    AG_REQUIRE(rows * cols == 0 || (x && bias && y), AG_ERR_INVALID_DIMS, "add: null pointer");
    AG_EW_ENTRY("add", add_bias_kernel, rows * cols, x, bias, y, rows * cols, cols);
}

extern "C" ag_status_t ag_add_broadcast_f32(ag_stream_t stream, const float *x, const float *b, float *y,
                                            const int *shape, const int *bshape, int rank)
{
    AG_REQUIRE(rank >= 1 && rank <= 8 && shape && bshape, AG_ERR_INVALID_DIMS, "add: rank %d not in 1..8", rank);
    size_t n = 1;
    for (int i = 0; i < rank; ++i) {
        AG_REQUIRE(shape[i] >= 0 && (bshape[i] == shape[i] || bshape[i] == 1), AG_ERR_INCOMPATIBLE_SHAPE,
                   "add: axis %d of the right operand has extent %d, the left %d", i, bshape[i], shape[i]);
        n *= (size_t)shape[i];
    }
    if (n == 0) return AG_OK;
    AG_REQUIRE(x && b && y, AG_ERR_INVALID_DIMS, "add: null pointer");
    // merge neighbours with the same broadcast state; axes of extent 1 join either kind
    BroadcastGeom g{};
    bool prev_bc = false;
    size_t bstride = 1;
    unsigned rev_dims[8], rev_bstride[8];
    int groups = 0;
    for (int i = rank - 1; i >= 0; --i) {
        if (shape[i] == 1) continue;
        const bool bc = bshape[i] == 1;
        if (groups > 0 && bc == prev_bc) {
            AG_REQUIRE((size_t)rev_dims[groups - 1] * (size_t)shape[i] <= 0xffffffffu, AG_ERR_INVALID_DIMS, "add: extent too large");
            rev_dims[groups - 1] *= (unsigned)shape[i];
        } else {
            rev_dims[groups] = (unsigned)shape[i];
            rev_bstride[groups] = bc ? 0u : (unsigned)bstride;
            ++groups;
        }
        if (!bc) bstride *= (size_t)shape[i];
        prev_bc = bc;
    }
    AG_REQUIRE(groups <= 6 && bstride <= 0xffffffffu, AG_ERR_INVALID_DIMS, "add: broadcast pattern with %d groups of axes not supported", groups);
    if (groups == 0) {
        rev_dims[0] = 1, rev_bstride[0] = 0, groups = 1;
    }
    g.rank = groups;
    for (int i = 0; i < groups; ++i) g.dims[i] = rev_dims[groups - 1 - i], g.bstride[i] = rev_bstride[groups - 1 - i];
    AG_EW_ENTRY("add", add_broadcast_kernel, n, x, b, y, n, g);
}

extern "C" ag_status_t ag_bias_grad_f32(ag_stream_t stream, const float *gy, float *out, size_t rows,
                                        size_t cols)
{
    AG_REQUIRE(cols == 0 || (out && (gy || rows == 0)), AG_ERR_INVALID_DIMS, "reduce_sum(axis 0): null pointer");
    if (cols == 0) return AG_OK;
    hipLaunchKernelGGL(bias_grad_kernel, dim3(ew_grid(cols, 1)), dim3(256), 0, as_stream(stream), gy, out,
                       rows, cols);
    return check_launch("reduce_sum(axis 0)");
}

extern "C" ag_status_t ag_add_n_f32(ag_stream_t stream, const float *const *xs, int count, float *out,
                                    size_t n)
{
    AG_REQUIRE(count >= 1 && count <= 8, AG_ERR_INVALID_DIMS, "add_n: between 1 and 8 inputs supported, got %d", count);
    AG_REQUIRE(xs && (n == 0 || out), AG_ERR_INVALID_DIMS, "add_n: null pointer");
    PtrPack pk{};
    for (int i = 0; i < count; ++i) {
        AG_REQUIRE(xs[i] || n == 0, AG_ERR_INVALID_DIMS, "add_n: input %d is null", i);
        pk.p[i] = xs[i];
    }
    AG_EW_ENTRY("add_n", add_n_kernel, n, pk, count, out, n);
}

extern "C" ag_status_t ag_mul_f32(ag_stream_t stream, const float *a, const float *b, float *out, size_t n)
{
    AG_REQUIRE(n == 0 || (a && b && out), AG_ERR_INVALID_DIMS, "mul: null pointer");
    AG_EW_ENTRY("mul", mul_kernel, n, a, b, out, n);
}

extern "C" ag_status_t ag_scale_f32(ag_stream_t stream, const float *a, float s, float *out, size_t n)
{
    AG_REQUIRE(n == 0 || (a && out), AG_ERR_INVALID_DIMS, "scale: null pointer");
    AG_EW_ENTRY("scale", scale_kernel, n, a, s, out, n);
}

extern "C" ag_status_t ag_div_scalar_f32(ag_stream_t stream, const float *a, float s, float *out, size_t n)
{
    AG_REQUIRE(n == 0 || (a && out), AG_ERR_INVALID_DIMS, "div: null pointer");
    AG_EW_ENTRY("div", div_scalar_kernel, n, a, s, out, n);
}

extern "C" ag_status_t ag_fill_f32(ag_stream_t stream, float *out, float value, size_t n)
{
    AG_REQUIRE(n == 0 || out, AG_ERR_INVALID_DIMS, "fill: null pointer");
    AG_EW_ENTRY("fill", fill_kernel, n, out, value, n);
}

extern "C" ag_status_t ag_sparse_softmax_xent_f32(ag_stream_t stream, const float *logits,
                                                  const float *labels, float *loss, float *log_softmax,
                                                  size_t rows, size_t classes)
{
    AG_REQUIRE(classes >= 1 || rows == 0, AG_ERR_INCOMPATIBLE_SHAPE,
               "SparseSoftmaxCrossEntropy: logits need at least one class");
    AG_REQUIRE(rows == 0 || (logits && labels && loss && log_softmax), AG_ERR_INVALID_DIMS,
               "SparseSoftmaxCrossEntropy: null pointer");
    if (rows == 0) return AG_OK;
    hipLaunchKernelGGL(sparse_xent_kernel, dim3(ew_grid(rows, 1)), dim3(256), 0, as_stream(stream), logits,
                       labels, loss, log_softmax, rows, classes);
    return check_launch("SparseSoftmaxCrossEntropy");
}

extern "C" ag_status_t ag_sparse_softmax_xent_grad_f32(ag_stream_t stream, const float *log_softmax,
                                                       const float *labels, const float *gy, float *gx,
                                                       size_t rows, size_t classes)
{
    AG_REQUIRE(rows * classes == 0 || (log_softmax && labels && gy && gx), AG_ERR_INVALID_DIMS,
               "SparseSoftmaxCrossEntropyGrad: null pointer");
    AG_EW_ENTRY("SparseSoftmaxCrossEntropyGrad", sparse_xent_grad_kernel, rows * classes, log_softmax,
                labels, gy, gx, rows, classes);
}
