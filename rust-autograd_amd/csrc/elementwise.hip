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

// Every streaming elementwise operator is a functor with `one(i)` (element i) and `vec(q)` (elements
// 4q..4q+3 through 128-bit streaming loads and stores).  With 16-byte aligned operands each thread
// of a one-shot grid handles one group of four, and one thread finishes a partial last group
// (copy-like kernels measured 6.2-6.7 TB/s this way on MI355X against 4.6-5.7 TB/s for scalar
// grid-strided loops); otherwise one element per thread, grid-strided.
template <typename F>
__global__ __launch_bounds__(256) void ew_vec_kernel(size_t n4, size_t n, F f)
{
    const size_t i = blockIdx.x * 256ull + threadIdx.x;
    if (i < n4) {
        f.vec(i);
    } else if (i == n4) {
        for (size_t e = n4 * 4; e < n; ++e) f.one(e);
    }
}

template <typename F>
__global__ __launch_bounds__(256) void ew_scalar_kernel(size_t n, F f)
{
    AG_EW_LOOP(i, n) f.one(i);
}

__device__ inline const float4 *as4(const float *p) { return reinterpret_cast<const float4 *>(p); }
__device__ inline float4 *as4(float *p) { return reinterpret_cast<float4 *>(p); }

// activation_ops.rs:155-159  x.max(0)  (f32::max: NaN input yields 0)
struct ReluF {
    const float *x;
    float *y;
    static __device__ float f(float v) { return v > 0.f ? v : 0.f; }
    __device__ void one(size_t i) const { y[i] = f(x[i]); }
    __device__ void vec(size_t q) const
    {
        const float4 v = ld_stream(as4(x) + q);
        st_stream(as4(y) + q, make_float4(f(v.x), f(v.y), f(v.z), f(v.w)));
    }
};

// activation_ops.rs:161-166  greater(x, 0) * gy
struct ReluGradF {
    const float *x, *gy;
    float *gx;
    static __device__ float f(float v, float g) { return (v > 0.f ? 1.f : 0.f) * g; }
    __device__ void one(size_t i) const { gx[i] = f(x[i], gy[i]); }
    __device__ void vec(size_t q) const
    {
        const float4 v = ld_stream(as4(x) + q), g = ld_stream(as4(gy) + q);
        st_stream(as4(gx) + q, make_float4(f(v.x, g.x), f(v.y, g.y), f(v.z, g.z), f(v.w, g.w)));
    }
};

struct PtrPack {
    const float *p[8];
};

// array_ops.rs:503-535  ((x0 + x1) + x2) + ...
struct AddNF {
    PtrPack xs;
    int count;
    float *out;
    __device__ void one(size_t i) const
    {
        float acc = xs.p[0][i];
        for (int j = 1; j < count; ++j) acc += xs.p[j][i];
        out[i] = acc;
    }
    __device__ void vec(size_t q) const
    {
        float4 acc = ld_stream(as4(xs.p[0]) + q);
        for (int j = 1; j < count; ++j) {
            const float4 v = ld_stream(as4(xs.p[j]) + q);
            acc.x += v.x;
            acc.y += v.y;
            acc.z += v.z;
            acc.w += v.w;
        }
        st_stream(as4(out) + q, acc);
    }
};

struct MulF {
    const float *a, *b;
    float *out;
    __device__ void one(size_t i) const { out[i] = a[i] * b[i]; }
    __device__ void vec(size_t q) const
    {
        const float4 u = ld_stream(as4(a) + q), v = ld_stream(as4(b) + q);
        st_stream(as4(out) + q, make_float4(u.x * v.x, u.y * v.y, u.z * v.z, u.w * v.w));
    }
};

template <bool DIVIDE>
struct ScaleF {
    const float *a;
    float s;
    float *out;
    __device__ float f(float v) const { return DIVIDE ? v / s : v * s; }
    __device__ void one(size_t i) const { out[i] = f(a[i]); }
    __device__ void vec(size_t q) const
    {
        const float4 v = ld_stream(as4(a) + q);
        st_stream(as4(out) + q, make_float4(f(v.x), f(v.y), f(v.z), f(v.w)));
    }
};

struct FillF {
    float *out;
    float v;
    __device__ void one(size_t i) const { out[i] = v; }
    __device__ void vec(size_t q) const { st_stream(as4(out) + q, make_float4(v, v, v, v)); }
};

// Broadcast of an operand `b` along its axes of extent 1.  `dims` are the result's extents after
// neighbouring axes with the same broadcast state have been merged (outermost first), `bstride` the
// stride of `b` for each merged axis in elements (0 where it is broadcast).
struct BroadcastGeom {
    unsigned dims[8];
    unsigned bstride[8];
    int rank;
};

// ADD: y = x + b (AddOp, binary_ops.rs:147-166, 304-346); otherwise y = b (ReduceGradCommon,
// reduction_ops.rs:459-512).  I = unsigned when the result has fewer than 2^32 elements.  `vec`
// needs an innermost merged extent that is a multiple of 4.
// MODE 0: y = broadcast(b); 1: y = x + broadcast(b); 2: y = relu(x + broadcast(b)), the sum rounded to f32 first,
// so the result has the bits of the two operations run one after the other.
template <int MODE, typename I>
struct BroadcastF {
    static __device__ float fin(float v) { return MODE == 2 ? ReluF::f(v) : v; }
    const float *x, *b;
    float *y;
    BroadcastGeom g;
    __device__ void one(size_t i) const
    {
        I rest = (I)i, bi = 0;
        for (int d = g.rank - 1; d > 0; --d) {
            const I q = rest / g.dims[d];
            bi += (rest - q * g.dims[d]) * g.bstride[d];
            rest = q;
        }
        bi += rest * g.bstride[0];
        y[i] = MODE != 0 ? fin(x[i] + b[bi]) : b[bi];
    }
    __device__ void vec(size_t q4) const
    {
        const int last = g.rank - 1;
        const I inner4 = g.dims[last] >> 2;
        I rest = (I)q4 / inner4;
        I bi = ((I)q4 - rest * inner4) * 4 * g.bstride[last];
        for (int d = last - 1; d > 0; --d) {
            const I q = rest / g.dims[d];
            bi += (rest - q * g.dims[d]) * g.bstride[d];
            rest = q;
        }
        if (last > 0) bi += rest * g.bstride[0];
        float4 bv;
        if (g.bstride[last] == 0) {
            const float s = b[bi];
            bv = make_float4(s, s, s, s);
        } else {
            bv = *reinterpret_cast<const float4 *>(b + bi);
        }
        if (MODE != 0) {
            const float4 v = ld_stream(as4(x) + q4);
            bv = make_float4(fin(v.x + bv.x), fin(v.y + bv.y), fin(v.z + bv.z), fin(v.w + bv.w));
        }
        st_stream(as4(y) + q4, bv);
    }
};

// out[c] = sum over rows, ascending (ndarray sum_axis(0) order used by MaybeReduceSum).
__global__ __launch_bounds__(256) void bias_grad_kernel(const float *__restrict__ gy,
                                                        float *__restrict__ out, size_t rows, size_t cols)
{
    AG_EW_LOOP(c, cols)
    {
        // eight loads in flight, added in row order
        float acc = 0.f;
        const float *p = gy + c;
        size_t r = 0;
        for (; r + 8 <= rows; r += 8, p += 8 * cols) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = p[u * cols];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += v[u];
        }
        for (; r < rows; ++r, p += cols) acc += *p;
        out[c] = acc;
    }
}

// A label is an f32 holding a class number (xent_ops.rs:96-104 casts it to usize and panics on a
// negative, non-finite or too large value: "can't cast to usize" / "Wrong label value").  A kernel
// cannot panic; such a row's loss and gradient are NaN instead, so the failure shows in the result.
__device__ inline bool label_of(float lf, size_t classes, size_t *label)
{
    const bool ok = lf >= 0.f && lf < (float)classes;  // false for NaN
    *label = ok ? (size_t)(int)lf : classes;
    return ok;
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
        size_t label;
        const bool ok = label_of(labels[r], classes, &label);
        float picked = 0.f;
        for (size_t c = 0; c < classes; ++c) {
            const float v = row[c] - lse;
            lsm[r * classes + c] = v;
            if (c == label) picked = v;
        }
        loss[r] = ok ? -picked : __builtin_nanf("");
    }
}

// The same arithmetic with the 256 rows of a block staged through LDS (row pitch odd, so the
// per-row scans are free of bank conflicts): global loads and stores are then contiguous across
// the wave instead of one row apart.  For up to 63 classes.
__global__ __launch_bounds__(256) void sparse_xent_lds_kernel(const float *__restrict__ logits,
                                                              const float *__restrict__ labels,
                                                              float *__restrict__ loss,
                                                              float *__restrict__ lsm, size_t rows,
                                                              unsigned classes, unsigned pitch)
{
    extern __shared__ float tile[];
    const size_t r0 = blockIdx.x * 256ull;
    const unsigned nrows = rows - r0 < 256 ? (unsigned)(rows - r0) : 256u;
    const unsigned count = nrows * classes;
    const float *src = logits + r0 * classes;
    float *dst = lsm + r0 * classes;
    for (unsigned e = threadIdx.x; e < count; e += 256) {
        const unsigned r = e / classes;
        tile[r * pitch + (e - r * classes)] = src[e];
    }
    __syncthreads();
    if (threadIdx.x < nrows) {
        float *row = tile + threadIdx.x * pitch;
        float mx = -FLT_MAX;
        for (unsigned c = 0; c < classes; ++c) mx = fmaxf(mx, row[c]);
        float s = 0.f;
        for (unsigned c = 0; c < classes; ++c) s += expf(row[c] - mx);
        const float lse = logf(s) + mx;
        size_t label;
        const bool ok = label_of(labels[r0 + threadIdx.x], classes, &label);
        float picked = 0.f;
        for (unsigned c = 0; c < classes; ++c) {
            const float v = row[c] - lse;
            row[c] = v;
            if (c == label) picked = v;
        }
        loss[r0 + threadIdx.x] = ok ? -picked : __builtin_nanf("");
    }
    __syncthreads();
    for (unsigned e = threadIdx.x; e < count; e += 256) {
        const unsigned r = e / classes;
        dst[e] = tile[r * pitch + (e - r * classes)];
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
        size_t label;
        const bool ok = label_of(labels[r], classes, &label);
        if (c == label) s -= 1.f;
        gx[i] = ok ? s * gy[r] : __builtin_nanf("");
    }
}

// The gradient straight from the logits: the log-softmax of sparse_xent_kernel and the arithmetic of
// sparse_xent_grad_kernel in one pass, one thread per row, so that a training step that never reads the loss does not
// run the forward kernel at all.  gy == null: every row's upstream gradient is gy_const.
__global__ __launch_bounds__(256) void sparse_xent_grad_logits_kernel(const float *__restrict__ logits,
                                                                      const float *__restrict__ labels,
                                                                      const float *__restrict__ gy, float gy_const,
                                                                      float *__restrict__ gx, size_t rows, size_t classes)
{
    AG_EW_LOOP(r, rows)
    {
        const float *row = logits + r * classes;
        float mx = -FLT_MAX;
        for (size_t c = 0; c < classes; ++c) mx = fmaxf(mx, row[c]);
        float s = 0.f;
        for (size_t c = 0; c < classes; ++c) s += expf(row[c] - mx);
        const float lse = logf(s) + mx;
        size_t label;
        const bool ok = label_of(labels[r], classes, &label);
        const float g = gy ? gy[r] : gy_const;
        for (size_t c = 0; c < classes; ++c) {
            float e = expf(row[c] - lse);
            if (c == label) e -= 1.f;
            gx[r * classes + c] = ok ? e * g : __builtin_nanf("");
        }
    }
}

}  // namespace ag

using namespace ag;

template <typename F>
static ag_status_t ew_launch(const char *name, ag_stream_t stream, size_t n, bool vec, const F &f)
{
    if (n == 0) return AG_OK;
    const size_t n4 = n / 4, blocks = (n4 + 256) / 256;  // n4 + 1 threads: the last finishes a partial group
    if (vec && blocks <= (size_t)kMaxGridX)
        hipLaunchKernelGGL((ew_vec_kernel<F>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), n4, n, f);
    else
        hipLaunchKernelGGL((ew_scalar_kernel<F>), dim3(ew_grid(n, 4)), dim3(256), 0, as_stream(stream), n, f);
    return check_launch(name);
}

// Merges neighbouring axes with the same broadcast state (axes of extent 1 join either kind).
static ag_status_t make_broadcast_geom(const char *who, const int *shape, const int *bshape, int rank,
                                       BroadcastGeom *g, size_t *n_out)
{
    AG_REQUIRE(rank >= 0 && rank <= 8 && (rank == 0 || (shape && bshape)), AG_ERR_INVALID_DIMS, "%s: rank %d not in 0..8", who, rank);
    size_t n = 1;
    for (int i = 0; i < rank; ++i) {
        AG_REQUIRE(shape[i] >= 0 && (bshape[i] == shape[i] || bshape[i] == 1), AG_ERR_INCOMPATIBLE_SHAPE,
                   "%s: axis %d of the broadcast operand has extent %d, the result %d", who, i, bshape[i], shape[i]);
        n *= (size_t)shape[i];
    }
    *n_out = n;
    bool prev_bc = false;
    size_t bstride = 1;
    unsigned rev_dims[8], rev_bstride[8];
    int groups = 0;
    for (int i = rank - 1; i >= 0; --i) {
        if (shape[i] == 1) continue;
        const bool bc = bshape[i] == 1;
        if (groups > 0 && bc == prev_bc) {
            AG_REQUIRE((size_t)rev_dims[groups - 1] * (size_t)shape[i] <= 0xffffffffu, AG_ERR_INVALID_DIMS, "%s: extent too large", who);
            rev_dims[groups - 1] *= (unsigned)shape[i];
        } else {
            rev_dims[groups] = (unsigned)shape[i];
            rev_bstride[groups] = bc ? 0u : (unsigned)bstride;
            ++groups;
        }
        if (!bc) bstride *= (size_t)shape[i];
        prev_bc = bc;
    }
    AG_REQUIRE(bstride <= 0xffffffffu, AG_ERR_INVALID_DIMS, "%s: operand too large", who);
    if (groups == 0) {
        rev_dims[0] = 1, rev_bstride[0] = 0, groups = 1;
    }
    g->rank = groups;
    for (int i = 0; i < groups; ++i) g->dims[i] = rev_dims[groups - 1 - i], g->bstride[i] = rev_bstride[groups - 1 - i];
    return AG_OK;
}

template <int MODE>
static ag_status_t launch_broadcast(const char *name, ag_stream_t stream, const float *x, const float *b, float *y,
                                    const BroadcastGeom &g, size_t n)
{
    const int last = g.rank - 1;
    const bool vec = g.dims[last] % 4 == 0 && aligned16(y) && (MODE == 0 || aligned16(x)) && (g.bstride[last] == 0 || aligned16(b));
    if (n <= 0xffffffffu) return ew_launch(name, stream, n, vec, BroadcastF<MODE, unsigned>{x, b, y, g});
    return ew_launch(name, stream, n, vec, BroadcastF<MODE, size_t>{x, b, y, g});
}

extern "C" ag_status_t ag_relu_f32(ag_stream_t stream, const float *x, float *y, size_t n)
{
    AG_REQUIRE(n == 0 || (x && y), AG_ERR_INVALID_DIMS, "relu: null pointer");
    return ew_launch("relu", stream, n, aligned16(x) && aligned16(y), ReluF{x, y});
}

extern "C" ag_status_t ag_relu_grad_f32(ag_stream_t stream, const float *x, const float *gy, float *gx,
                                        size_t n)
{
    AG_REQUIRE(n == 0 || (x && gy && gx), AG_ERR_INVALID_DIMS, "relu_grad: null pointer");
    return ew_launch("relu_grad", stream, n, aligned16(x) && aligned16(gy) && aligned16(gx), ReluGradF{x, gy, gx});
}

extern "C" ag_status_t ag_add_bias_f32(ag_stream_t stream, const float *x, const float *bias, float *y,
                                       size_t rows, size_t cols)
{
    AG_REQUIRE(rows * cols == 0 || (x && bias && y), AG_ERR_INVALID_DIMS, "add: null pointer");
    AG_REQUIRE(rows <= 0x7fffffffu && cols <= 0x7fffffffu, AG_ERR_INVALID_DIMS, "add: extent too large");
    const int shape[2] = {(int)rows, (int)cols}, bshape[2] = {1, (int)cols};
    BroadcastGeom g{};
    size_t n;
    if (ag_status_t s = make_broadcast_geom("add", shape, bshape, 2, &g, &n)) return s;
    if (n == 0) return AG_OK;
    return launch_broadcast<1>("add", stream, x, bias, y, g, n);
}

extern "C" ag_status_t ag_add_broadcast_f32(ag_stream_t stream, const float *x, const float *b, float *y,
                                            const int *shape, const int *bshape, int rank)
{
    AG_REQUIRE(rank >= 1, AG_ERR_INVALID_DIMS, "add: rank %d not in 1..8", rank);
    BroadcastGeom g{};
    size_t n;
    if (ag_status_t s = make_broadcast_geom("add", shape, bshape, rank, &g, &n)) return s;
    if (n == 0) return AG_OK;
    AG_REQUIRE(x && b && y, AG_ERR_INVALID_DIMS, "add: null pointer");
    return launch_broadcast<1>("add", stream, x, b, y, g, n);
}

extern "C" ag_status_t ag_add_broadcast_relu_f32(ag_stream_t stream, const float *x, const float *b, float *y,
                                                 const int *shape, const int *bshape, int rank)
{
    AG_REQUIRE(rank >= 1, AG_ERR_INVALID_DIMS, "add+relu: rank %d not in 1..8", rank);
    BroadcastGeom g{};
    size_t n;
    if (ag_status_t s = make_broadcast_geom("add+relu", shape, bshape, rank, &g, &n)) return s;
    if (n == 0) return AG_OK;
    AG_REQUIRE(x && b && y, AG_ERR_INVALID_DIMS, "add+relu: null pointer");
    return launch_broadcast<2>("add+relu", stream, x, b, y, g, n);
}

extern "C" ag_status_t ag_broadcast_grad_f32(ag_stream_t stream, const float *gy, float *gx,
                                             const int *shape, int rank, const int *axes, int n_axes)
{
    int sorted[8], bshape[8];
    if (ag_status_t s = check_axes("reduce_grad", shape, rank, axes, n_axes, sorted)) return s;
    for (int d = 0; d < rank; ++d) bshape[d] = shape[d];
    for (int j = 0; j < n_axes; ++j) bshape[sorted[j]] = 1;
    BroadcastGeom g{};
    size_t n;
    if (ag_status_t s = make_broadcast_geom("reduce_grad", shape, bshape, rank, &g, &n)) return s;
    if (n == 0) return AG_OK;
    AG_REQUIRE(gy && gx, AG_ERR_INVALID_DIMS, "reduce_grad: null pointer");
    return launch_broadcast<0>("reduce_grad", stream, nullptr, gy, gx, g, n);
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
    AddNF f{};
    bool vec = aligned16(out);
    for (int i = 0; i < count; ++i) {
        AG_REQUIRE(xs[i] || n == 0, AG_ERR_INVALID_DIMS, "add_n: input %d is null", i);
        f.xs.p[i] = xs[i];
        vec = vec && aligned16(xs[i]);
    }
    f.count = count;
    f.out = out;
    return ew_launch("add_n", stream, n, vec, f);
}

extern "C" ag_status_t ag_mul_f32(ag_stream_t stream, const float *a, const float *b, float *out, size_t n)
{
    AG_REQUIRE(n == 0 || (a && b && out), AG_ERR_INVALID_DIMS, "mul: null pointer");
    return ew_launch("mul", stream, n, aligned16(a) && aligned16(b) && aligned16(out), MulF{a, b, out});
}

extern "C" ag_status_t ag_scale_f32(ag_stream_t stream, const float *a, float s, float *out, size_t n)
{
    AG_REQUIRE(n == 0 || (a && out), AG_ERR_INVALID_DIMS, "scale: null pointer");
    return ew_launch("scale", stream, n, aligned16(a) && aligned16(out), ScaleF<false>{a, s, out});
}

extern "C" ag_status_t ag_div_scalar_f32(ag_stream_t stream, const float *a, float s, float *out, size_t n)
{
    AG_REQUIRE(n == 0 || (a && out), AG_ERR_INVALID_DIMS, "div: null pointer");
    return ew_launch("div", stream, n, aligned16(a) && aligned16(out), ScaleF<true>{a, s, out});
}

extern "C" ag_status_t ag_fill_f32(ag_stream_t stream, float *out, float value, size_t n)
{
    AG_REQUIRE(n == 0 || out, AG_ERR_INVALID_DIMS, "fill: null pointer");
    return ew_launch("fill", stream, n, aligned16(out), FillF{out, value});
}

#define AG_EW_ENTRY(name, kernel, nexpr, ...)                                                     \
    do {                                                                                          \
        const size_t n__ = (nexpr);                                                               \
        if (n__ == 0) return AG_OK;                                                               \
        hipLaunchKernelGGL(kernel, dim3(ew_grid(n__, 4)), dim3(256), 0, as_stream(stream), __VA_ARGS__); \
        return check_launch(name);                                                                \
    } while (0)

extern "C" ag_status_t ag_sparse_softmax_xent_f32(ag_stream_t stream, const float *logits,
                                                  const float *labels, float *loss, float *log_softmax,
                                                  size_t rows, size_t classes)
{
    AG_REQUIRE(classes >= 1 || rows == 0, AG_ERR_INCOMPATIBLE_SHAPE,
               "SparseSoftmaxCrossEntropy: logits need at least one class");
    AG_REQUIRE(rows == 0 || (logits && labels && loss && log_softmax), AG_ERR_INVALID_DIMS,
               "SparseSoftmaxCrossEntropy: null pointer");
    if (rows == 0) return AG_OK;
    if (classes <= 63 && (rows + 255) / 256 <= (size_t)kMaxGridX) {
        const unsigned pitch = (unsigned)classes | 1u;
        hipLaunchKernelGGL(sparse_xent_lds_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 256 * pitch * sizeof(float),
                           as_stream(stream), logits, labels, loss, log_softmax, rows, (unsigned)classes, pitch);
        return check_launch("SparseSoftmaxCrossEntropy");
    }
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

// SparseSoftmaxCrossEntropy's gradient without its forward (xent_ops.rs:63-115 and 139-153 in one kernel): the bits of
// ag_sparse_softmax_xent_f32 followed by ag_sparse_softmax_xent_grad_f32.  gy [rows] may be NULL: then every row's
// upstream gradient is gy_const (the mean of a batch loss: 1 / rows).
extern "C" ag_status_t ag_sparse_softmax_xent_grad_logits_f32(ag_stream_t stream, const float *logits, const float *labels,
                                                              const float *gy, float gy_const, float *gx, size_t rows,
                                                              size_t classes)
{
    AG_REQUIRE(classes >= 1 || rows == 0, AG_ERR_INCOMPATIBLE_SHAPE,
               "SparseSoftmaxCrossEntropyGrad: logits need at least one class");
    AG_REQUIRE(rows == 0 || (logits && labels && gx), AG_ERR_INVALID_DIMS, "SparseSoftmaxCrossEntropyGrad: null pointer");
    if (rows == 0) return AG_OK;
    hipLaunchKernelGGL(sparse_xent_grad_logits_kernel, dim3(ew_grid(rows, 1)), dim3(256), 0, as_stream(stream), logits, labels,
                       gy, gy_const, gx, rows, classes);
    return check_launch("SparseSoftmaxCrossEntropyGrad");
}
