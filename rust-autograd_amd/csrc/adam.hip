// Fused Adam update: one pass over param / grad / m / v (28 bytes of HBM traffic per element)
// instead of the reference's seven array passes and two temporaries
// (gradient_descent_ops/adam.rs:11-58).  The arithmetic keeps the reference's operation order
// with contraction into fused multiply-adds switched off, so m and v match it bit for bit.
#include "ag_internal.h"

namespace ag {

struct AdamCoef {
    float alpha, eps, b1, b2;
};

__device__ inline void adam_one(float &p, float g, float &m, float &v, float c1, float c2, float rm,
                                float rv, const AdamCoef &k)
{
// Every multiply and add below is rounded on its own, as in the reference (no fused multiply-add);
// this file is also compiled with -ffp-contract=off.
#pragma clang fp contract(off)
    m = m * k.b1 + c1 * g;               // adam.rs:16-23
    v = v * k.b2 + c2 * g * g;           // adam.rs:26-33   ((1-b2)*g)*g
    const float vh = v * rv;             // adam.rs:38-39   v * (1/(1-b2^t))
    float mh = m * rm;                   // adam.rs:40-41   m * (1/(1-b1^t))
    mh = mh / (sqrtf(vh) + k.eps);       // adam.rs:44      correctly rounded sqrt and divide
    p = p - k.alpha * mh;                // adam.rs:49-50
}

// One 128-bit quad per thread (no loop: the grid covers the array, which measured fastest for a
// streaming read-modify-write); the two bias-correction factors are computed by one lane per
// block and shared through LDS.  The last partial quad is handled by the final thread.
// `block` is the block's index within this parameter's share of the grid.
__device__ inline void adam_block(float *__restrict__ p, const float *__restrict__ g, float *__restrict__ m,
                                  float *__restrict__ v, const float *__restrict__ t, size_t n,
                                  const AdamCoef &k, int vec, size_t block)
{
    __shared__ float corr[2];
    if (threadIdx.x == 0) {
        const float tv = t[0];
        corr[0] = 1.0f / (1.0f - powf(k.b1, tv));  // adam.rs:40
        corr[1] = 1.0f / (1.0f - powf(k.b2, tv));  // adam.rs:38
    }
    __syncthreads();
    const float rm = corr[0], rv = corr[1];
    const float c1 = 1.0f - k.b1, c2 = 1.0f - k.b2;
    const size_t i = block * 256ull + threadIdx.x;
    if (vec) {
        const size_t n4 = n / 4;
        if (i < n4) {
            float4 pp = ld_stream(reinterpret_cast<const float4 *>(p) + i);
            float4 mm = ld_stream(reinterpret_cast<const float4 *>(m) + i);
            float4 vv = ld_stream(reinterpret_cast<const float4 *>(v) + i);
            const float4 gg = ld_stream(reinterpret_cast<const float4 *>(g) + i);
            adam_one(pp.x, gg.x, mm.x, vv.x, c1, c2, rm, rv, k);
            adam_one(pp.y, gg.y, mm.y, vv.y, c1, c2, rm, rv, k);
            adam_one(pp.z, gg.z, mm.z, vv.z, c1, c2, rm, rv, k);
            adam_one(pp.w, gg.w, mm.w, vv.w, c1, c2, rm, rv, k);
            st_stream(reinterpret_cast<float4 *>(p) + i, pp);
            st_stream(reinterpret_cast<float4 *>(m) + i, mm);
            st_stream(reinterpret_cast<float4 *>(v) + i, vv);
        } else if (i == n4) {
            for (size_t e = n4 * 4; e < n; ++e) {
                float pp = p[e], mm = m[e], vv = v[e];
                adam_one(pp, g[e], mm, vv, c1, c2, rm, rv, k);
                p[e] = pp;
                m[e] = mm;
                v[e] = vv;
            }
        }
    } else if (i < n) {
        float pp = p[i], mm = m[i], vv = v[i];
        adam_one(pp, g[i], mm, vv, c1, c2, rm, rv, k);
        p[i] = pp;
        m[i] = mm;
        v[i] = vv;
    }
}

// Large arrays: a block walks a contiguous run of kAdamRun chunks (one chunk = one quad per thread = 4 KiB per array)
// with its seven streams skewed in time.  In step s it loads g of chunk s, m of chunk s-1, v of chunk s-2 and p of
// chunk s-3, updates chunk s-4, and stores p of chunk s-4, m of chunk s-5 and v of chunk s-6: at any instant the
// streams of a thread are 4 KiB apart.  The one-quad-per-thread form above touches element i of all four arrays at
// once, and where the caller's arrays all start on a 2 MiB boundary (what hipMalloc hands out) those four addresses
// fall into the same DRAM bank -- four rows of one bank opened in turn: 2^26 elements took 0.358 ms that way and
// 0.317 ms with the arrays 4 KiB apart modulo 2 MiB; this form takes 0.323 ms wherever they are (runs of 2 / 3 / 4 / 5 /
// 6 / 8 / 16 / 32 chunks: 0.333 / 0.331 / 0.323 / 0.328 / 0.329 / 0.327 / 0.345 / 0.359 ms with aligned arrays --
// short runs keep more blocks, and with them more independent streams, in flight).  Same arithmetic per element,
// so the same bits.
constexpr int kAdamRun = 4;
constexpr size_t kAdamRunFrom = (size_t)1 << 20;  // elements from which the run form is used

// `block` < adam_full_runs(n): every chunk of the run lies inside the array (no bounds tests: with them the
// compiler waits for every outstanding load and store at each step).
__device__ inline void adam_block_run(float *__restrict__ p, const float *__restrict__ g, float *__restrict__ m,
                                      float *__restrict__ v, const float *__restrict__ t, const AdamCoef &k, size_t block)
{
    __shared__ float corr[2];
    if (threadIdx.x == 0) {
        const float tv = t[0];
        corr[0] = 1.0f / (1.0f - powf(k.b1, tv));  // adam.rs:40
        corr[1] = 1.0f / (1.0f - powf(k.b2, tv));  // adam.rs:38
    }
    __syncthreads();
    const float rm = corr[0], rv = corr[1];
    const float c1 = 1.0f - k.b1, c2 = 1.0f - k.b2;
    const size_t q0 = block * (size_t)(kAdamRun * 256) + threadIdx.x;  // this thread's quad of chunk 0
    const float4 *g4 = reinterpret_cast<const float4 *>(g) + q0;
    float4 *p4 = reinterpret_cast<float4 *>(p) + q0, *m4 = reinterpret_cast<float4 *>(m) + q0,
           *v4 = reinterpret_cast<float4 *>(v) + q0;
    float4 G[kAdamRun], M[kAdamRun], V[kAdamRun], P[kAdamRun];  // (registers: after unrolling each lives for a few steps)
#pragma unroll
    for (int s = 0; s < kAdamRun + 7; ++s) {
        // this step's loads first; the chunk updated below was loaded in earlier steps, so the wait in front of its
        // arithmetic leaves these loads (and the previous step's stores) in flight
        if (s < kAdamRun) G[s] = ld_stream(g4 + s * 256);
        if (s >= 1 && s - 1 < kAdamRun) M[s - 1] = ld_stream(m4 + (s - 1) * 256);
        if (s >= 2 && s - 2 < kAdamRun) V[s - 2] = ld_stream(v4 + (s - 2) * 256);
        if (s >= 3 && s - 3 < kAdamRun) P[s - 3] = ld_stream(p4 + (s - 3) * 256);
        if (s >= 4 && s - 4 < kAdamRun) {
            const int c = s - 4;
            adam_one(P[c].x, G[c].x, M[c].x, V[c].x, c1, c2, rm, rv, k);
            adam_one(P[c].y, G[c].y, M[c].y, V[c].y, c1, c2, rm, rv, k);
            adam_one(P[c].z, G[c].z, M[c].z, V[c].z, c1, c2, rm, rv, k);
            adam_one(P[c].w, G[c].w, M[c].w, V[c].w, c1, c2, rm, rv, k);
            st_stream(p4 + c * 256, P[c]);
        }
        if (s >= 5 && s - 5 < kAdamRun) st_stream(m4 + (s - 5) * 256, M[s - 5]);
        if (s >= 6 && s - 6 < kAdamRun) st_stream(v4 + (s - 6) * 256, V[s - 6]);
        __builtin_amdgcn_sched_barrier(0);  // the steps stay in this order: the skew between the streams is the point
    }
}

// Whole runs of a large array (`vec` == 2) go to the run form, what is left (and every smaller or unaligned
// array) to the one-quad-per-thread form.
__host__ __device__ inline size_t adam_full_runs(size_t n) { return n / 4 / (size_t)(kAdamRun * 256); }
inline size_t adam_blocks(size_t n, int vec)
{
    if (n == 0) return 0;
    if (vec != 2) return ((vec ? n / 4 + 1 : n) + 255) / 256;  // +1: the thread that finishes a partial quad
    const size_t full = adam_full_runs(n), rest = n - full * (size_t)(kAdamRun * 1024);
    return full + (rest / 4 + 1 + 255) / 256;
}
__device__ inline void adam_entry(float *__restrict__ p, const float *__restrict__ g, float *__restrict__ m,
                                  float *__restrict__ v, const float *__restrict__ t, size_t n, const AdamCoef &k, int vec,
                                  size_t block)
{
    if (vec == 2) {
        const size_t full = adam_full_runs(n);
        if (block < full) {
            adam_block_run(p, g, m, v, t, k, block);
        } else {
            const size_t off = full * (size_t)(kAdamRun * 1024);
            adam_block(p + off, g + off, m + off, v + off, t, n - off, k, 1, block - full);
        }
    } else {
        adam_block(p, g, m, v, t, n, k, vec, block);
    }
}

__global__ __launch_bounds__(256) void adam_kernel(float *__restrict__ p, const float *__restrict__ g,
                                                   float *__restrict__ m, float *__restrict__ v,
                                                   const float *__restrict__ t, size_t n, AdamCoef k,
                                                   int vec)
{
    adam_entry(p, g, m, v, t, n, k, vec, blockIdx.x);
}

// Several parameters in one launch: the table travels in the kernel arguments, each parameter owns
// the blocks [first_block[i], first_block[i+1]).  Per element the arithmetic is adam_block's, so
// the results equal those of one adam_kernel launch per parameter.
constexpr int kAdamMultiMax = 24;
struct AdamTable {
    float *p[kAdamMultiMax];
    const float *g[kAdamMultiMax];
    float *m[kAdamMultiMax];
    float *v[kAdamMultiMax];
    float *t[kAdamMultiMax];
    unsigned long long n[kAdamMultiMax];
    unsigned first_block[kAdamMultiMax + 1];
    int vec[kAdamMultiMax];
    int count;
};

__global__ __launch_bounds__(256) void adam_multi_kernel(AdamTable tab, AdamCoef k)
{
    int i = 0;
    while (i + 1 < tab.count && blockIdx.x >= tab.first_block[i + 1]) ++i;
    adam_entry(tab.p[i], tab.g[i], tab.m[i], tab.v[i], tab.t[i], (size_t)tab.n[i], k, tab.vec[i], blockIdx.x - tab.first_block[i]);
}

// t += 1 for every parameter of the table, after the update kernel has read them (same stream => ordered)
__global__ void adam_tick_multi_kernel(AdamTable tab)
{
    const int i = threadIdx.x;
    if (i < tab.count) tab.t[i][0] = tab.t[i][0] + 1.0f;
}

// t += 1 after every update kernel of this step has read it (same stream => ordered).  adam.rs:52-54
__global__ void adam_tick_kernel(float *t) { t[0] = t[0] + 1.0f; }

}  // namespace ag

using namespace ag;

extern "C" ag_status_t ag_adam_update_f32(ag_stream_t stream, float *param, const float *grad, float *m,
                                          float *v, float *t, size_t n, float alpha, float eps, float b1,
                                          float b2)
{
    AG_REQUIRE(t, AG_ERR_INVALID_DIMS, "adam: null step counter");
    AG_REQUIRE(n == 0 || (param && grad && m && v), AG_ERR_INVALID_DIMS, "adam: null pointer");
    hipStream_t st = as_stream(stream);
    if (n > 0) {
        int vec = aligned16(param) && aligned16(grad) && aligned16(m) && aligned16(v);
        if (vec && n >= kAdamRunFrom) vec = 2;
        const size_t blocks = adam_blocks(n, vec);
        AG_REQUIRE(blocks <= (size_t)kMaxGridX, AG_ERR_INVALID_DIMS, "adam: too many elements (%zu)", n);
        hipLaunchKernelGGL(adam_kernel, dim3((unsigned)blocks), dim3(256), 0, st, param, grad, m, v, t, n,
                           AdamCoef{alpha, eps, b1, b2}, vec);
    }
    hipLaunchKernelGGL(adam_tick_kernel, dim3(1), dim3(1), 0, st, t);
    return check_launch("adam");
}

extern "C" int ag_adam_update_multi_max(void) { return kAdamMultiMax; }

extern "C" ag_status_t ag_adam_update_multi_f32(ag_stream_t stream, int count, float *const *params,
                                                const float *const *grads, float *const *ms, float *const *vs,
                                                float *const *ts, const size_t *ns, float alpha, float eps,
                                                float b1, float b2)
{
    AG_REQUIRE(count >= 0 && count <= kAdamMultiMax, AG_ERR_INVALID_DIMS, "adam: %d parameters in one call (at most %d)",
               count, kAdamMultiMax);
    if (count == 0) return AG_OK;
    AG_REQUIRE(params && grads && ms && vs && ts && ns, AG_ERR_INVALID_DIMS, "adam: null pointer table");
    AdamTable tab = {};
    tab.count = count;
    size_t total = 0;
    for (int i = 0; i < count; ++i) {
        AG_REQUIRE(ts[i], AG_ERR_INVALID_DIMS, "adam: null step counter (parameter %d)", i);
        AG_REQUIRE(ns[i] == 0 || (params[i] && grads[i] && ms[i] && vs[i]), AG_ERR_INVALID_DIMS,
                   "adam: null pointer (parameter %d)", i);
        for (int j = 0; j < i; ++j)
            AG_REQUIRE(ts[j] != ts[i] && (ns[i] == 0 || ns[j] == 0 || (params[j] != params[i] && ms[j] != ms[i] && vs[j] != vs[i])),
                       AG_ERR_INVALID_DIMS, "adam: parameters %d and %d share an array; update them in separate calls", j, i);
        // a gradient that another entry of the same launch writes (its param, m or v) would be read while it changes
        for (int j = 0; j < count; ++j)
            AG_REQUIRE(j == i || ns[i] == 0 || ns[j] == 0 ||
                           (grads[i] != params[j] && grads[i] != ms[j] && grads[i] != vs[j]),
                       AG_ERR_INVALID_DIMS,
                       "adam: the gradient of parameter %d is an array that parameter %d updates; update them in separate calls", i, j);
        int vec = aligned16(params[i]) && aligned16(grads[i]) && aligned16(ms[i]) && aligned16(vs[i]);
        if (vec && ns[i] >= kAdamRunFrom) vec = 2;
        tab.p[i] = params[i];
        tab.g[i] = grads[i];
        tab.m[i] = ms[i];
        tab.v[i] = vs[i];
        tab.t[i] = ts[i];
        tab.n[i] = ns[i];
        tab.vec[i] = vec;
        tab.first_block[i] = (unsigned)total;
        total += adam_blocks(ns[i], vec);
        AG_REQUIRE(total <= (size_t)kMaxGridX, AG_ERR_INVALID_DIMS, "adam: too many elements in one call");
    }
    tab.first_block[count] = (unsigned)total;
    hipStream_t st = as_stream(stream);
    if (total > 0)
        hipLaunchKernelGGL(adam_multi_kernel, dim3((unsigned)total), dim3(256), 0, st, tab, AdamCoef{alpha, eps, b1, b2});
    hipLaunchKernelGGL(adam_tick_multi_kernel, dim3(1), dim3(64), 0, st, tab);
    return check_launch("adam");
}
