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
__global__ __launch_bounds__(256) void adam_kernel(float *__restrict__ p, const float *__restrict__ g,
                                                   float *__restrict__ m, float *__restrict__ v,
                                                   const float *__restrict__ t, size_t n, AdamCoef k,
                                                   int vec)
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
    const size_t i = blockIdx.x * 256ull + threadIdx.x;
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
