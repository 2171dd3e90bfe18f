// reduce_sum / reduce_mean / sum-to-scalar and the broadcast their gradients need.
//
// HBM-bound.  Whole-array sums run in two deterministic stages: a fixed grid of blocks each
// accumulates a grid-strided slice with 128-bit loads, folds it with wave64 shuffles and an LDS
// step, and writes one partial; one block then folds the partials in index order.  Axis
// reductions are applied one axis at a time from the last listed axis to the first, exactly as
// the reference does (reduction_ops.rs:74-89).  With trailing elements after the folded axis
// (inner > 1), or a short folded axis, each thread owns one output and adds along the axis
// sequentially, which is the reference's own order (bit-identical sums); a long innermost axis
// uses one wave per row instead (tolerance-level agreement).
#include "ag_internal.h"

namespace ag {

constexpr int kSumBlocks = 2048;  // stage-1 partials (fixed: result does not depend on the device)
constexpr int kSumThreads = 256;
constexpr int kMaxRank = 8;
constexpr size_t kSeqRowLimit = 256;  // innermost folds up to this length are added sequentially

__device__ inline float wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    return v;
}

// Block-wide sum; valid in thread 0.
__device__ inline float block_sum(float v, float *lds)
{
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) lds[wave] = v;
    __syncthreads();
    float r = 0.f;
    if (threadIdx.x == 0)
        for (int w = 0; w < (int)(blockDim.x >> 6); ++w) r += lds[w];
    return r;
}

__global__ __launch_bounds__(kSumThreads) void sum_stage1_kernel(const float *__restrict__ x,
                                                                 size_t n, float *__restrict__ partial)
{
    __shared__ float lds[kSumThreads / 64];
    const size_t tid = blockIdx.x * (size_t)kSumThreads + threadIdx.x;
    const size_t nthreads = (size_t)gridDim.x * kSumThreads;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    const bool vec = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    size_t done = 0;
    if (vec) {
        const size_t n4 = n / 4;
        const float4 *x4 = reinterpret_cast<const float4 *>(x);
        size_t i = tid;
        // four independent 128-bit loads in flight per thread
        for (; i + 3 * nthreads < n4; i += 4 * nthreads) {
            const float4 v0 = ld_stream(x4 + i), v1 = ld_stream(x4 + i + nthreads), v2 = ld_stream(x4 + i + 2 * nthreads),
                         v3 = ld_stream(x4 + i + 3 * nthreads);
            a0 += (v0.x + v1.x) + (v2.x + v3.x);
            a1 += (v0.y + v1.y) + (v2.y + v3.y);
            a2 += (v0.z + v1.z) + (v2.z + v3.z);
            a3 += (v0.w + v1.w) + (v2.w + v3.w);
        }
        for (; i < n4; i += nthreads) {
            const float4 v = x4[i];
            a0 += v.x;
            a1 += v.y;
            a2 += v.z;
            a3 += v.w;
        }
        done = n4 * 4;
    }
    for (size_t i = done + tid; i < n; i += nthreads) a0 += x[i];
    const float s = block_sum((a0 + a1) + (a2 + a3), lds);
    if (threadIdx.x == 0) partial[blockIdx.x] = s;
}

__global__ __launch_bounds__(kSumThreads) void sum_stage2_kernel(const float *__restrict__ partial,
                                                                 int count, float scale,
                                                                 float *__restrict__ out)
{
    __shared__ float lds[kSumThreads / 64];
    float a = 0.f;
    for (int i = threadIdx.x; i < count; i += kSumThreads) a += partial[i];
    const float s = block_sum(a, lds);
    if (threadIdx.x == 0) out[0] = s * scale;
}

// x [outer][len][inner] -> out [outer][inner], inner > 1: sequential along `len` per thread.
__global__ __launch_bounds__(256) void fold_axis_seq_kernel(const float *__restrict__ x,
                                                            float *__restrict__ out, size_t outer,
                                                            size_t len, size_t inner, float scale,
                                                            int apply_scale)
{
    const size_t total = outer * inner;
    for (size_t t = blockIdx.x * 256ull + threadIdx.x; t < total; t += gridDim.x * 256ull) {
        const size_t o = t / inner, i = t - o * inner;
        const float *p = x + o * len * inner + i;
        float acc = 0.f;
        for (size_t r = 0; r < len; ++r) acc += p[r * inner];
        out[t] = apply_scale ? acc * scale : acc;
    }
}

// Long axis, few outputs: x [outer][len][inner] -> part [outer][splits][inner]; split s adds rows
// [s*chunk, min(len, (s+1)*chunk)) sequentially.  A second fold_axis_seq_kernel over the `splits`
// axis finishes the sum (fixed order, deterministic; rounding differs from one long chain).
__global__ __launch_bounds__(256) void fold_axis_split_kernel(const float *__restrict__ x,
                                                              float *__restrict__ part, size_t outer,
                                                              size_t len, size_t inner, size_t splits,
                                                              size_t chunk)
{
    const size_t total = outer * splits * inner;
    for (size_t t = blockIdx.x * 256ull + threadIdx.x; t < total; t += gridDim.x * 256ull) {
        const size_t i = t % inner, os = t / inner;
        const size_t sp = os % splits, o = os / splits;
        const size_t r0 = sp * chunk, r1 = min(len, r0 + chunk);
        const float *p = x + (o * len + r0) * inner + i;
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
        size_t r = r0;
        for (; r + 3 < r1; r += 4) {  // four independent loads in flight
            a0 += p[0];
            a1 += p[inner];
            a2 += p[2 * inner];
            a3 += p[3 * inner];
            p += 4 * inner;
        }
        for (; r < r1; ++r, p += inner) a0 += p[0];
        part[t] = (a0 + a1) + (a2 + a3);
    }
}

// x [rows][len] -> out [rows]: one wave per row, lanes stride the row, shuffle fold.
__global__ __launch_bounds__(256) void fold_last_axis_kernel(const float *__restrict__ x,
                                                             float *__restrict__ out, size_t rows,
                                                             size_t len, float scale, int apply_scale)
{
    const int lane = threadIdx.x & 63;
    const size_t wave = (blockIdx.x * 256ull + threadIdx.x) >> 6;
    const size_t nwaves = (gridDim.x * 256ull) >> 6;
    for (size_t r = wave; r < rows; r += nwaves) {
        const float *p = x + r * len;
        float acc = 0.f;
        for (size_t i = lane; i < len; i += 64) acc += p[i];
        acc = wave_sum(acc);
        if (lane == 0) out[r] = apply_scale ? acc * scale : acc;
    }
}

__global__ __launch_bounds__(256) void scale_copy_kernel(const float *__restrict__ x,
                                                         float *__restrict__ out, size_t n, float scale,
                                                         int apply_scale)
{
    for (size_t i = blockIdx.x * 256ull + threadIdx.x; i < n; i += gridDim.x * 256ull)
        out[i] = apply_scale ? x[i] * scale : x[i];
}

struct BroadcastShape {
    int rank;
    int dim[kMaxRank];       // extents of gx
    long long gstride[kMaxRank];  // stride of that axis inside gy (0 for reduced axes)
};

__global__ __launch_bounds__(256) void broadcast_kernel(const float *__restrict__ gy,
                                                        float *__restrict__ gx, BroadcastShape s,
                                                        size_t total)
{
    for (size_t flat = blockIdx.x * 256ull + threadIdx.x; flat < total; flat += gridDim.x * 256ull) {
        size_t rem = flat;
        long long src = 0;
        for (int d = s.rank - 1; d >= 0; --d) {
            const size_t c = rem % (size_t)s.dim[d];
            rem /= (size_t)s.dim[d];
            src += (long long)c * s.gstride[d];
        }
        gx[flat] = gy[src];
    }
}

// Split a long fold with few outputs so that the whole chip takes part.  Returns the number of
// splits (1 = no split) and the rows per split.
static size_t fold_splits(size_t outer, size_t len, size_t inner, size_t *chunk)
{
    *chunk = len;
    if (inner <= 1 || len < 1024 || outer * inner >= 262144) return 1;
    size_t want = 1048576 / (outer * inner);  // aim at ~1 M threads
    if (want > len / 64) want = len / 64;
    if (want < 2) return 1;
    *chunk = (len + want - 1) / want;
    return (len + *chunk - 1) / *chunk;
}

static unsigned grid_for(size_t work_items, int per_block)
{
    size_t b = (work_items + per_block - 1) / per_block;
    if (b < 1) b = 1;
    if (b > 65536) b = 65536;
    return (unsigned)b;
}

static ag_status_t check_axes(const char *who, const int *shape, int rank, const int *axes, int n_axes,
                              int *sorted)
{
    AG_REQUIRE(rank >= 0 && rank <= kMaxRank, AG_ERR_INVALID_DIMS, "%s: rank %d not in [0,%d]", who, rank, kMaxRank);
    AG_REQUIRE(n_axes >= 0 && n_axes <= rank, AG_ERR_INVALID_DIMS, "%s: %d axes for rank %d", who, n_axes, rank);
    for (int i = 0; i < rank; ++i)
        AG_REQUIRE(shape[i] >= 0, AG_ERR_INVALID_DIMS, "%s: negative extent %d at axis %d", who, shape[i], i);
    for (int i = 0; i < n_axes; ++i) {
        AG_REQUIRE(axes[i] >= 0 && axes[i] < rank, AG_ERR_OUT_OF_BOUNDS, "%s: axis %d out of range for rank %d",
                   who, axes[i], rank);
        sorted[i] = axes[i];
    }
    for (int i = 1; i < n_axes; ++i)
        for (int j = i; j > 0 && sorted[j - 1] > sorted[j]; --j) {
            const int t = sorted[j];
            sorted[j] = sorted[j - 1];
            sorted[j - 1] = t;
        }
    for (int i = 1; i < n_axes; ++i)
        AG_REQUIRE(sorted[i] != sorted[i - 1], AG_ERR_INVALID_DIMS, "%s: axis %d listed twice", who, sorted[i]);
    return AG_OK;
}

}  // namespace ag

using namespace ag;

extern "C" size_t ag_sum_all_f32_workspace(size_t n)
{
    (void)n;
    return sizeof(float) * kSumBlocks;
}

extern "C" ag_status_t ag_sum_all_f32(ag_stream_t stream, const float *x, size_t n, float *out,
                                      void *ws, size_t ws_bytes)
{
    AG_REQUIRE(out, AG_ERR_INVALID_DIMS, "sum_all: null output");
    AG_REQUIRE(ws && ws_bytes >= ag_sum_all_f32_workspace(n), AG_ERR_INVALID_DIMS,
               "sum_all: workspace of %zu bytes needed, %zu given", ag_sum_all_f32_workspace(n), ws_bytes);
    AG_REQUIRE(x || n == 0, AG_ERR_INVALID_DIMS, "sum_all: null input");
    float *partial = static_cast<float *>(ws);
    size_t blocks = (n + kSumThreads * 16 - 1) / (kSumThreads * 16);
    if (blocks < 1) blocks = 1;
    if (blocks > kSumBlocks) blocks = kSumBlocks;
    hipLaunchKernelGGL(sum_stage1_kernel, dim3((unsigned)blocks), dim3(kSumThreads), 0, as_stream(stream),
                       x, n, partial);
    hipLaunchKernelGGL(sum_stage2_kernel, dim3(1), dim3(kSumThreads), 0, as_stream(stream), partial,
                       (int)blocks, 1.0f, out);
    return check_launch("sum_all");
}

// Workspace layout: two ping-pong buffers for the intermediate results of multi-axis reductions
// (each as large as the result of the first fold) followed by the partials of a split fold.
static void reduce_ws_layout(const int *shape, int rank, const int *sorted_axes, int n_axes, size_t *pingpong,
                             size_t *split_floats)
{
    *pingpong = 0;
    *split_floats = 0;
    if (n_axes <= 0 || rank <= 0) return;
    size_t total = 1;
    int dims[kMaxRank];
    for (int i = 0; i < rank; ++i) {
        dims[i] = shape[i];
        total *= (size_t)shape[i];
    }
    if (n_axes > 1) {
        const int last = sorted_axes[n_axes - 1];
        size_t first = shape[last] ? total / (size_t)shape[last] : 0;
        if (first < 1) first = 1;
        *pingpong = (first + 3) & ~(size_t)3;
    }
    for (int a = n_axes - 1; a >= 0; --a) {
        size_t outer = 1, inner = 1, chunk;
        for (int i = 0; i < sorted_axes[a]; ++i) outer *= (size_t)dims[i];
        for (int i = sorted_axes[a] + 1; i < rank; ++i) inner *= (size_t)dims[i];
        const size_t sp = fold_splits(outer, (size_t)dims[sorted_axes[a]], inner, &chunk);
        if (sp > 1 && sp * outer * inner > *split_floats) *split_floats = sp * outer * inner;
        dims[sorted_axes[a]] = 1;
    }
}

extern "C" size_t ag_reduce_sum_f32_workspace(const int *shape, int rank, const int *axes, int n_axes)
{
    int ax[kMaxRank];
    if (rank < 0 || rank > kMaxRank || n_axes < 0 || n_axes > rank) return 16;
    for (int i = 0; i < n_axes; ++i) {
        if (axes[i] < 0 || axes[i] >= rank) return 16;
        ax[i] = axes[i];
    }
    for (int i = 1; i < n_axes; ++i)
        for (int j = i; j > 0 && ax[j - 1] > ax[j]; --j) {
            const int t = ax[j];
            ax[j] = ax[j - 1];
            ax[j - 1] = t;
        }
    size_t pp, sf;
    reduce_ws_layout(shape, rank, ax, n_axes, &pp, &sf);
    return sizeof(float) * (2 * pp + sf) + 32;
}

extern "C" ag_status_t ag_reduce_sum_f32(ag_stream_t stream, const float *x, float *out,
                                         const int *shape, int rank, const int *axes, int n_axes,
                                         int mean, void *ws, size_t ws_bytes)
{
    int ax[kMaxRank];
    if (ag_status_t s = check_axes(mean ? "reduce_mean" : "reduce_sum", shape, rank, axes, n_axes, ax)) return s;
    size_t total = 1;
    int dims[kMaxRank];
    for (int i = 0; i < rank; ++i) {
        dims[i] = shape[i];
        total *= (size_t)shape[i];
    }
    // reduced length accumulated in f32 and applied as a reciprocal (reduction_ops.rs:198-209)
    float red_len = 1.f;
    for (int i = 0; i < n_axes; ++i) red_len *= (float)shape[ax[i]];
    const float scale = 1.0f / red_len;
    const int do_scale = mean && n_axes > 0;
    size_t out_n = 1;
    for (int i = 0; i < rank; ++i) {
        bool red = false;
        for (int j = 0; j < n_axes; ++j) red |= ax[j] == i;
        if (!red) out_n *= (size_t)shape[i];
    }
    if (out_n == 0) return AG_OK;
    AG_REQUIRE(out && (x || total == 0), AG_ERR_INVALID_DIMS, "reduce_sum: null pointer");
    hipStream_t st = as_stream(stream);
    if (n_axes == 0 || rank == 0) {  // nothing to fold: the reference returns a view of x
        hipLaunchKernelGGL(scale_copy_kernel, dim3(grid_for(total, 256)), dim3(256), 0, st, x, out, total,
                           1.f, 0);
        return check_launch("reduce_sum");
    }
    size_t pp, sf;
    reduce_ws_layout(shape, rank, ax, n_axes, &pp, &sf);
    const size_t need = sizeof(float) * (2 * pp + sf);
    AG_REQUIRE(need == 0 || (ws && ws_bytes >= need), AG_ERR_INVALID_DIMS,
               "reduce_sum: workspace of %zu bytes needed, %zu given", need, ws_bytes);
    float *buf[2] = {static_cast<float *>(ws), static_cast<float *>(ws) + pp};
    float *part = static_cast<float *>(ws) + 2 * pp;
    const float *cur = x;
    for (int a = n_axes - 1; a >= 0; --a) {
        size_t outer = 1, inner = 1, chunk;
        for (int i = 0; i < ax[a]; ++i) outer *= (size_t)dims[i];
        for (int i = ax[a] + 1; i < rank; ++i) inner *= (size_t)dims[i];
        const size_t len = (size_t)dims[ax[a]];
        float *dst = (a == 0) ? out : buf[(n_axes - 1 - a) & 1];
        const int sc = (a == 0) ? do_scale : 0;
        const size_t sp = fold_splits(outer, len, inner, &chunk);
        // Short innermost folds stay sequential per output (the reference's order, bit-identical);
        // long rows take one wave each; long folds with few outputs are split over the chip.
        if (inner == 1 && len > kSeqRowLimit) {
            hipLaunchKernelGGL(fold_last_axis_kernel, dim3(grid_for(outer, 4)), dim3(256), 0, st, cur, dst,
                               outer, len, scale, sc);
        } else if (sp > 1) {
            hipLaunchKernelGGL(fold_axis_split_kernel, dim3(grid_for(outer * sp * inner, 256)), dim3(256), 0, st,
                               cur, part, outer, len, inner, sp, chunk);
            hipLaunchKernelGGL(fold_axis_seq_kernel, dim3(grid_for(outer * inner, 256)), dim3(256), 0, st, part,
                               dst, outer, sp, inner, scale, sc);
        } else {
            hipLaunchKernelGGL(fold_axis_seq_kernel, dim3(grid_for(outer * inner, 256)), dim3(256), 0, st, cur,
                               dst, outer, len, inner, scale, sc);
        }
        dims[ax[a]] = 1;
        cur = dst;
    }
    return check_launch(mean ? "reduce_mean" : "reduce_sum");
}

extern "C" ag_status_t ag_broadcast_grad_f32(ag_stream_t stream, const float *gy, float *gx,
                                             const int *shape, int rank, const int *axes, int n_axes)
{
    int ax[kMaxRank];
    if (ag_status_t s = check_axes("reduce_grad", shape, rank, axes, n_axes, ax)) return s;
    BroadcastShape bs;
    bs.rank = rank;
    size_t total = 1;
    long long stride = 1;
    for (int d = rank - 1; d >= 0; --d) {
        bool red = false;
        for (int j = 0; j < n_axes; ++j) red |= ax[j] == d;
        bs.dim[d] = shape[d];
        bs.gstride[d] = red ? 0 : stride;
        if (!red) stride *= shape[d];
        total *= (size_t)shape[d];
    }
    if (total == 0) return AG_OK;
    AG_REQUIRE(gy && gx, AG_ERR_INVALID_DIMS, "reduce_grad: null pointer");
    hipLaunchKernelGGL(broadcast_kernel, dim3(grid_for(total, 256)), dim3(256), 0, as_stream(stream), gy,
                       gx, bs, total);
    return check_launch("reduce_grad");
}
