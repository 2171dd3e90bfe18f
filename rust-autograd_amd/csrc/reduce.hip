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
//
// Inputs of 2^20 elements and more take the streaming folds instead: neighbouring axes with the
// same state are merged, the last folded group goes first (it reads the whole input, every later
// step a small intermediate), and every step keeps many independent 128-bit streaming loads in
// flight per thread over contiguous memory -- a group of lanes per row for a trailing group, a
// thread per output column (split along the folded axis until the chip is full) otherwise.  Sums
// agree with the sequential order to rounding.
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
        // Each block streams one contiguous run of the input, eight 128-bit loads in flight per
        // thread: measured 7.0 TB/s on MI355X against 5.4 TB/s for loads a whole grid apart.
        const size_t n4 = n / 4;
        const float4 *x4 = reinterpret_cast<const float4 *>(x);
        const size_t per_block = (n4 + gridDim.x - 1) / gridDim.x;
        const size_t b0 = blockIdx.x * per_block;
        const size_t b1 = b0 + per_block < n4 ? b0 + per_block : n4;
        size_t i = b0 + threadIdx.x;
        constexpr int U = 8;
        for (; i + (U - 1) * kSumThreads < b1; i += U * kSumThreads) {
            float4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = ld_stream(x4 + i + u * kSumThreads);
#pragma unroll
            for (int u = 0; u < U; u += 2) {
                a0 += v[u].x + v[u + 1].x;
                a1 += v[u].y + v[u + 1].y;
                a2 += v[u].z + v[u + 1].z;
                a3 += v[u].w + v[u + 1].w;
            }
        }
        for (; i < b1; i += kSumThreads) {
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
        size_t r = 0;
        for (; r + 8 <= len; r += 8, p += 8 * inner) {  // eight loads in flight, added in axis order
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = p[u * inner];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += v[u];
        }
        for (; r < len; ++r, p += inner) acc += *p;
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

// ---- streaming folds (large inputs) ------------------------------------------------------------

// x [rows][len] -> out [rows]: G lanes per row, rows of one wave adjacent in memory.
template <int G, bool VEC>
__global__ __launch_bounds__(256) void fold_rows_kernel(const float *__restrict__ x, float *__restrict__ out,
                                                        size_t rows, size_t len, float scale, int apply_scale)
{
    const unsigned lane = threadIdx.x % G;
    const size_t row = (blockIdx.x * 256ull + threadIdx.x) / G;
    const bool live = row < rows;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    if (live) {
        const float *p = x + row * len;
        if (VEC) {
            const float4 *p4 = reinterpret_cast<const float4 *>(p);
            const size_t len4 = len / 4;
            size_t j = lane;
            for (; j + 3 * G < len4; j += 4 * G) {
                const float4 v0 = ld_stream(p4 + j), v1 = ld_stream(p4 + j + G), v2 = ld_stream(p4 + j + 2 * G),
                             v3 = ld_stream(p4 + j + 3 * G);
                a0 += (v0.x + v1.x) + (v2.x + v3.x);
                a1 += (v0.y + v1.y) + (v2.y + v3.y);
                a2 += (v0.z + v1.z) + (v2.z + v3.z);
                a3 += (v0.w + v1.w) + (v2.w + v3.w);
            }
            for (; j < len4; j += G) {
                const float4 v = ld_stream(p4 + j);
                a0 += v.x;
                a1 += v.y;
                a2 += v.z;
                a3 += v.w;
            }
        } else {
            size_t j = lane;
            for (; j + 3 * G < len; j += 4 * G) {
                a0 += ld_stream(p + j);
                a1 += ld_stream(p + j + G);
                a2 += ld_stream(p + j + 2 * G);
                a3 += ld_stream(p + j + 3 * G);
            }
            for (; j < len; j += G) a0 += ld_stream(p + j);
        }
    }
    float s = (a0 + a1) + (a2 + a3);
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) s += __shfl_down(s, off, G);
    if (live && lane == 0) out[row] = apply_scale ? s * scale : s;
}

// Few long rows: x [rows][len] -> part [rows][splits]; block (row, split) streams elements
// [split*chunk, min(len, (split+1)*chunk)) of its row (chunk a multiple of 4).
template <bool VEC>
__global__ __launch_bounds__(256) void fold_rows_split_kernel(const float *__restrict__ x, float *__restrict__ part,
                                                              size_t len, unsigned splits, size_t chunk)
{
    __shared__ float lds[4];
    const size_t row = blockIdx.x / splits;
    const unsigned sp = blockIdx.x % splits;
    const size_t e0 = (size_t)sp * chunk, e1 = e0 + chunk < len ? e0 + chunk : len;
    const float *p = x + row * len;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    if (VEC) {
        const float4 *p4 = reinterpret_cast<const float4 *>(p);
        const size_t q1 = e1 / 4;
        size_t i = e0 / 4 + threadIdx.x;
        constexpr int U = 8;
        for (; i + (U - 1) * 256 < q1; i += U * 256) {
            float4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = ld_stream(p4 + i + u * 256);
#pragma unroll
            for (int u = 0; u < U; u += 2) {
                a0 += v[u].x + v[u + 1].x;
                a1 += v[u].y + v[u + 1].y;
                a2 += v[u].z + v[u + 1].z;
                a3 += v[u].w + v[u + 1].w;
            }
        }
        for (; i < q1; i += 256) {
            const float4 v = ld_stream(p4 + i);
            a0 += v.x;
            a1 += v.y;
            a2 += v.z;
            a3 += v.w;
        }
    } else {
        size_t i = e0 + threadIdx.x;
        for (; i + 3 * 256 < e1; i += 4 * 256) {
            a0 += ld_stream(p + i);
            a1 += ld_stream(p + i + 256);
            a2 += ld_stream(p + i + 512);
            a3 += ld_stream(p + i + 768);
        }
        for (; i < e1; i += 256) a0 += ld_stream(p + i);
    }
    const float s = block_sum((a0 + a1) + (a2 + a3), lds);
    if (threadIdx.x == 0) part[blockIdx.x] = s;
}

template <typename T>
__device__ inline T vec_zero();
template <>
__device__ inline float vec_zero<float>() { return 0.f; }
template <>
__device__ inline float4 vec_zero<float4>() { return make_float4(0.f, 0.f, 0.f, 0.f); }
__device__ inline float vadd(float a, float b) { return a + b; }
__device__ inline float4 vadd(const float4 &a, const float4 &b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }
__device__ inline float vscale(float a, float s) { return a * s; }
__device__ inline float4 vscale(const float4 &a, float s) { return make_float4(a.x * s, a.y * s, a.z * s, a.w * s); }

// x [outer][len][inner] -> out [outer][splits][inner], T = float4 when inner is a multiple of 4:
// one thread per output column (of T), rows [split*chunk, min(len, (split+1)*chunk)) added with
// eight loads in flight.  grid = (column blocks, splits, min(outer, 65535)).
template <typename T>
__global__ __launch_bounds__(256) void fold_cols_kernel(const float *__restrict__ x, float *__restrict__ out,
                                                        size_t outer, size_t len, size_t inner_t, size_t chunk,
                                                        float scale, int apply_scale)
{
    const size_t col = blockIdx.x * 256ull + threadIdx.x;
    if (col >= inner_t) return;
    const unsigned sp = blockIdx.y, splits = gridDim.y;
    const size_t r0 = (size_t)sp * chunk, r1 = r0 + chunk < len ? r0 + chunk : len;
    for (size_t o = blockIdx.z; o < outer; o += gridDim.z) {
        const T *p = reinterpret_cast<const T *>(x) + (o * len + r0) * inner_t + col;
        T acc0 = vec_zero<T>(), acc1 = vec_zero<T>();
        size_t r = r0;
        constexpr int U = 8;
        for (; r + U <= r1; r += U) {
            T v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = ld_stream(p + u * inner_t);
            acc0 = vadd(acc0, vadd(vadd(v[0], v[1]), vadd(v[2], v[3])));
            acc1 = vadd(acc1, vadd(vadd(v[4], v[5]), vadd(v[6], v[7])));
            p += U * inner_t;
        }
        for (; r < r1; ++r, p += inner_t) acc0 = vadd(acc0, ld_stream(p));
        T sum = vadd(acc0, acc1);
        if (apply_scale) sum = vscale(sum, scale);
        reinterpret_cast<T *>(out)[(o * splits + sp) * inner_t + col] = sum;
    }
}

// x [outer][len][inner] -> out [outer][inner] in ONE pass for inner a multiple of four: a block takes 32
// column quads and splits the rows over its eight groups of 32 lanes (eight 128-bit loads in flight per
// lane); the group sums meet in LDS and are added in group order, so the result is deterministic.
// Compared with a thread per column plus a second pass over split partial sums this needs one launch,
// writes no partials, and has eight times the lanes per column.
__global__ __launch_bounds__(256) void fold_cols_groups_kernel(const float *__restrict__ x, float *__restrict__ out,
                                                               size_t outer, size_t len, size_t inner4, float scale,
                                                               int apply_scale)
{
    __shared__ float4 part[8][32];
    const unsigned c = threadIdx.x & 31, g = threadIdx.x >> 5;
    const size_t col = blockIdx.x * 32ull + c;
    const size_t chunk = (len + 7) / 8;
    const size_t r0 = (size_t)g * chunk < len ? (size_t)g * chunk : len, r1 = r0 + chunk < len ? r0 + chunk : len;
    for (size_t o = blockIdx.y; o < outer; o += gridDim.y) {
        float4 acc0 = vec_zero<float4>(), acc1 = vec_zero<float4>();
        if (col < inner4) {
            const float4 *p = reinterpret_cast<const float4 *>(x) + (o * len + r0) * inner4 + col;
            size_t r = r0;
            constexpr int U = 8;
            for (; r + U <= r1; r += U) {
                float4 v[U];
#pragma unroll
                for (int u = 0; u < U; ++u) v[u] = ld_stream(p + u * inner4);
                acc0 = vadd(acc0, vadd(vadd(v[0], v[1]), vadd(v[2], v[3])));
                acc1 = vadd(acc1, vadd(vadd(v[4], v[5]), vadd(v[6], v[7])));
                p += U * inner4;
            }
            for (; r < r1; ++r, p += inner4) acc0 = vadd(acc0, ld_stream(p));
        }
        part[g][c] = vadd(acc0, acc1);
        __syncthreads();
        if (g == 0 && col < inner4) {
            float4 sum = part[0][c];
#pragma unroll
            for (int g2 = 1; g2 < 8; ++g2) sum = vadd(sum, part[g2][c]);
            if (apply_scale) sum = vscale(sum, scale);
            reinterpret_cast<float4 *>(out)[o * inner4 + col] = sum;
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(256) void scale_copy_kernel(const float *__restrict__ x,
                                                         float *__restrict__ out, size_t n, float scale,
                                                         int apply_scale)
{
    for (size_t i = blockIdx.x * 256ull + threadIdx.x; i < n; i += gridDim.x * 256ull)
        out[i] = apply_scale ? x[i] * scale : x[i];
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

ag_status_t check_axes(const char *who, const int *shape, int rank, const int *axes, int n_axes,
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

// ---- plan of the streaming folds -----------------------------------------------------------------
constexpr size_t kStreamMinElements = (size_t)1 << 20;
constexpr size_t kStreamBlocks = 2048;  // blocks a fold is split into, at least, when its shape allows

struct StreamStep {
    int kind;  // 0: lanes per row; 1: blocks per row, then 0 over the partials; 2: thread per column
    size_t outer, len, inner;
    unsigned splits;
    size_t chunk;
};
struct StreamPlan {
    int n_steps;
    StreamStep step[kMaxRank];
    bool scalar;      // every element is folded: the whole-array sum
    size_t pingpong;  // floats of each of the two intermediate buffers
    size_t partial;   // floats for the partial sums of split folds
};

static size_t ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }

static void plan_step(StreamStep *st)
{
    st->splits = 1;
    st->chunk = st->len;
    if (st->inner == 1) {
        st->kind = 0;
        if (st->len >= 16384 && st->outer < kStreamBlocks) {
            size_t sp = ceil_div(kStreamBlocks, st->outer);
            if (sp > st->len / 4096) sp = st->len / 4096;
            if (sp >= 2) {
                st->kind = 1;
                st->chunk = (ceil_div(st->len, sp) + 3) & ~(size_t)3;
                st->splits = (unsigned)ceil_div(st->len, st->chunk);
            }
        }
    } else {
        st->kind = 2;
        const size_t inner_t = st->inner % 4 == 0 ? st->inner / 4 : st->inner;
        const size_t blocks = ceil_div(inner_t, 256) * (st->outer < 65535 ? st->outer : 65535);
        size_t sp = ceil_div(kStreamBlocks, blocks);
        if (sp > st->len / 16) sp = st->len / 16;
        if (sp > 65535) sp = 65535;
        if (sp >= 2) {
            st->chunk = ceil_div(st->len, sp);
            st->splits = (unsigned)ceil_div(st->len, st->chunk);
        }
    }
}

// False when the input is small or nothing is folded: the sequential folds handle those.
static bool plan_stream(const int *shape, int rank, const int *sorted_axes, int n_axes, StreamPlan *pl)
{
    size_t total = 1;
    for (int i = 0; i < rank; ++i) total *= (size_t)shape[i];
    if (n_axes == 0 || total < kStreamMinElements) return false;
    size_t ext[kMaxRank];
    bool red[kMaxRank];
    int ng = 0;
    bool any = false;
    for (int i = 0; i < rank; ++i) {
        if (shape[i] == 1) continue;
        bool r = false;
        for (int j = 0; j < n_axes; ++j) r |= sorted_axes[j] == i;
        any |= r;
        if (ng > 0 && red[ng - 1] == r) {
            ext[ng - 1] *= (size_t)shape[i];
        } else {
            ext[ng] = (size_t)shape[i];
            red[ng] = r;
            ++ng;
        }
    }
    if (!any) return false;
    pl->n_steps = 0;
    pl->pingpong = pl->partial = 0;
    pl->scalar = ng == 1;
    if (pl->scalar) {
        pl->partial = kSumBlocks;
        return true;
    }
    for (;;) {
        int j = -1, left = 0;
        for (int g = 0; g < ng; ++g)
            if (red[g]) {
                j = g;
                ++left;
            }
        if (j < 0) break;
        StreamStep st{};
        st.outer = st.inner = 1;
        for (int g = 0; g < j; ++g) st.outer *= ext[g];
        for (int g = j + 1; g < ng; ++g) st.inner *= ext[g];
        st.len = ext[j];
        plan_step(&st);
        const size_t result = st.outer * st.inner;
        if (left > 1 && ((result + 3) & ~(size_t)3) > pl->pingpong) pl->pingpong = (result + 3) & ~(size_t)3;
        if (st.splits > 1 && result * st.splits > pl->partial) pl->partial = result * st.splits;
        pl->step[pl->n_steps++] = st;
        // drop the folded group; the kept groups on either side become one
        int w = 0;
        for (int g = 0; g < ng; ++g) {
            if (g == j) continue;
            if (w > 0 && red[w - 1] == red[g]) {
                ext[w - 1] *= ext[g];
            } else {
                ext[w] = ext[g];
                red[w] = red[g];
                ++w;
            }
        }
        ng = w;
    }
    return true;
}

static void launch_fold_rows(hipStream_t st, const float *src, float *dst, size_t rows, size_t len, float scale, int sc)
{
    const bool vec = len % 4 == 0 && aligned16(src);
    const size_t lanes = vec ? len / 4 : len;
    const int G = lanes >= 32 ? 64 : lanes >= 8 ? 16 : 4;
    const dim3 grid((unsigned)ceil_div(rows * (size_t)G, 256)), block(256);
#define AG_FOLD_ROWS(GG)                                                                                               \
    do {                                                                                                               \
        if (vec) hipLaunchKernelGGL((fold_rows_kernel<GG, true>), grid, block, 0, st, src, dst, rows, len, scale, sc);  \
        else hipLaunchKernelGGL((fold_rows_kernel<GG, false>), grid, block, 0, st, src, dst, rows, len, scale, sc);     \
    } while (0)
    if (G == 64) AG_FOLD_ROWS(64);
    else if (G == 16) AG_FOLD_ROWS(16);
    else AG_FOLD_ROWS(4);
#undef AG_FOLD_ROWS
}

static void launch_fold_cols(hipStream_t st, const float *src, float *dst, size_t outer, size_t len, size_t inner,
                             unsigned splits, size_t chunk, float scale, int sc)
{
    const bool vec = inner % 4 == 0 && aligned16(src) && aligned16(dst);
    const size_t inner_t = vec ? inner / 4 : inner;
    const dim3 grid((unsigned)ceil_div(inner_t, 256), splits, (unsigned)(outer < 65535 ? outer : 65535)), block(256);
    if (vec) hipLaunchKernelGGL((fold_cols_kernel<float4>), grid, block, 0, st, src, dst, outer, len, inner_t, chunk, scale, sc);
    else hipLaunchKernelGGL((fold_cols_kernel<float>), grid, block, 0, st, src, dst, outer, len, inner_t, chunk, scale, sc);
}

static void run_stream(hipStream_t st, const StreamPlan &pl, const float *x, size_t total, float *out, float *ws,
                       float scale, int do_scale)
{
    float *buf[2] = {ws, ws + pl.pingpong};
    float *part = ws + 2 * pl.pingpong;
    if (pl.scalar) {
        size_t blocks = ceil_div(total, kSumThreads * 16);
        if (blocks > (size_t)kSumBlocks) blocks = kSumBlocks;
        hipLaunchKernelGGL(sum_stage1_kernel, dim3((unsigned)blocks), dim3(kSumThreads), 0, st, x, total, part);
        hipLaunchKernelGGL(sum_stage2_kernel, dim3(1), dim3(kSumThreads), 0, st, part, (int)blocks,
                           do_scale ? scale : 1.0f, out);
        return;
    }
    const float *cur = x;
    for (int i = 0; i < pl.n_steps; ++i) {
        const StreamStep &s = pl.step[i];
        const bool last = i == pl.n_steps - 1;
        float *dst = last ? out : buf[i & 1];
        const int sc = last ? do_scale : 0;
        if (s.kind == 0) {
            launch_fold_rows(st, cur, dst, s.outer, s.len, scale, sc);
        } else if (s.kind == 1) {
            const bool vec = s.len % 4 == 0 && aligned16(cur);
            const dim3 grid((unsigned)(s.outer * s.splits)), block(256);
            if (vec) hipLaunchKernelGGL((fold_rows_split_kernel<true>), grid, block, 0, st, cur, part, s.len, s.splits, s.chunk);
            else hipLaunchKernelGGL((fold_rows_split_kernel<false>), grid, block, 0, st, cur, part, s.len, s.splits, s.chunk);
            launch_fold_rows(st, part, dst, s.outer, s.splits, scale, sc);
        } else if (s.inner % 4 == 0 && s.len >= 16 && aligned16(cur) && aligned16(dst)) {
            const size_t inner4 = s.inner / 4;
            const dim3 grid((unsigned)ceil_div(inner4, 32), (unsigned)(s.outer < 65535 ? s.outer : 65535));
            hipLaunchKernelGGL(fold_cols_groups_kernel, grid, dim3(256), 0, st, cur, dst, s.outer, s.len, inner4, scale, sc);
        } else if (s.splits > 1) {
            launch_fold_cols(st, cur, part, s.outer, s.len, s.inner, s.splits, s.chunk, 1.f, 0);
            launch_fold_cols(st, part, dst, s.outer, s.splits, s.inner, 1, s.splits, scale, sc);
        } else {
            launch_fold_cols(st, cur, dst, s.outer, s.len, s.inner, 1, s.len, scale, sc);
        }
        cur = dst;
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
    size_t floats = 2 * pp + sf;
    StreamPlan pl;
    if (plan_stream(shape, rank, ax, n_axes, &pl) && 2 * pl.pingpong + pl.partial > floats) floats = 2 * pl.pingpong + pl.partial;
    return sizeof(float) * floats + 32;
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
    StreamPlan pl;
    if (plan_stream(shape, rank, ax, n_axes, &pl)) {
        const size_t need = sizeof(float) * (2 * pl.pingpong + pl.partial);
        AG_REQUIRE(need == 0 || (ws && ws_bytes >= need), AG_ERR_INVALID_DIMS,
                   "reduce_sum: workspace of %zu bytes needed, %zu given", need, ws_bytes);
        bool fits = true;  // launch limits of the streaming kernels
        for (int i = 0; i < pl.n_steps; ++i) {
            const StreamStep &s = pl.step[i];
            const size_t blocks = s.kind == 0 ? ceil_div(s.outer, 4) : s.kind == 1 ? s.outer * s.splits : ceil_div(s.inner, 256);
            fits &= blocks < (size_t)kMaxGridX;
        }
        if (fits) {
            run_stream(st, pl, x, total, out, static_cast<float *>(ws), scale, do_scale);
            return check_launch(mean ? "reduce_mean" : "reduce_sum");
        }
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
