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

__global__ __launch_bounds__(256) void adam_kernel(float *__restrict__ p, const float *__restrict__ g,
                                                   float *__restrict__ m, float *__restrict__ v,
                                                   const float *__restrict__ t, size_t n, AdamCoef k,
                                                   int vec)
{
    adam_block(p, g, m, v, t, n, k, vec, blockIdx.x);
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
    adam_block(tab.p[i], tab.g[i], tab.m[i], tab.v[i], tab.t[i], (size_t)tab.n[i], k, tab.vec[i],
               blockIdx.x - tab.first_block[i]);
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
        const int vec = aligned16(param) && aligned16(grad) && aligned16(m) && aligned16(v);
        const size_t items = vec ? n / 4 + 1 : n;  // +1: the thread that finishes a partial quad
        const size_t blocks = (items + 255) / 256;
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
        const int vec = aligned16(params[i]) && aligned16(grads[i]) && aligned16(ms[i]) && aligned16(vs[i]);
        const size_t items = ns[i] == 0 ? 0 : (vec ? ns[i] / 4 + 1 : ns[i]);
        tab.p[i] = params[i];
        tab.g[i] = grads[i];
        tab.m[i] = ms[i];
        tab.v[i] = vs[i];
        tab.t[i] = ts[i];
        tab.n[i] = ns[i];
        tab.vec[i] = vec;
        tab.first_block[i] = (unsigned)total;
        total += (items + 255) / 256;
        AG_REQUIRE(total <= (size_t)kMaxGridX, AG_ERR_INVALID_DIMS, "adam: too many elements in one call");
    }
    tab.first_block[count] = (unsigned)total;
    hipStream_t st = as_stream(stream);
    if (total > 0)
        hipLaunchKernelGGL(adam_multi_kernel, dim3((unsigned)total), dim3(256), 0, st, tab, AdamCoef{alpha, eps, b1, b2});
    hipLaunchKernelGGL(adam_tick_multi_kernel, dim3(1), dim3(64), 0, st, tab);
    return check_launch("adam");
}
