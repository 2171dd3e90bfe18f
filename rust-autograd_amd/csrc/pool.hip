// MaxPool2D forward, argmax backward and the argmax gather used by the second-order op.
//
// All three are HBM-bound elementwise-style kernels over NCHW planes.  The backward is written
// as a gather: each input pixel visits the (few) windows that contain it in ascending (oy, ox)
// order and adds the upstream gradient of those that selected it.  That is the order in which
// the reference's sequential scatter `gx[argmax[i]] += gy[i]` (max_pool2d.rs:123-131) reaches the
// pixel, so sums are bit-identical and no atomics or zero-fill pass are needed.
#include <cfloat>

#include "ag_internal.h"

namespace ag {

struct PoolGeom {
    int H, W, OH, OW, size, stride;
};

__global__ __launch_bounds__(256) void maxpool_fwd_kernel(const float *__restrict__ x,
                                                          float *__restrict__ y,
                                                          float *__restrict__ argmax,
                                                          int32_t *__restrict__ idx_local,
                                                          PoolGeom g, int chunks)
{
    const int chunk = blockIdx.x % chunks;
    const long long plane = blockIdx.x / chunks;
    const int o = chunk * 256 + threadIdx.x;
    if (o >= g.OH * g.OW) return;
    const int oy = o / g.OW, ox = o - oy * g.OW;
    const int h0 = oy * g.stride, w0 = ox * g.stride;
    const int h1 = min(h0 + g.size, g.H), w1 = min(w0 + g.size, g.W);
    const long long base = plane * (long long)g.H * g.W;
    const float *xp = x + base;
    // Start value and tie rule of max_pool2d.rs:51-70: most negative finite float, index 0,
    // replaced only by a strictly greater value (NaN never wins).
    float best = -FLT_MAX;
    int best_local = -1;
    for (int h = h0; h < h1; ++h)
        for (int w = w0; w < w1; ++w) {
            const float v = xp[h * g.W + w];
            if (v > best) {
                best = v;
                best_local = h * g.W + w;
            }
        }
    const long long out = plane * (long long)g.OH * g.OW + o;
    y[out] = best;
    // The reference stores the whole-tensor offset converted to f32 by value (max_pool2d.rs:74-75).
    const unsigned long long flat = best_local >= 0 ? (unsigned long long)(base + best_local) : 0ull;
    argmax[out] = (float)flat;  // round-to-nearest-even, like Rust's `as f32`
    if (idx_local) idx_local[out] = best_local;
}

// EXACT: selection read from the plane-local int32 buffer; otherwise from the f32 argmax.
template <bool EXACT>
__global__ __launch_bounds__(256) void maxpool_bwd_kernel(const float *__restrict__ gy,
                                                          const float *__restrict__ argmax,
                                                          const int32_t *__restrict__ idx_local,
                                                          float *__restrict__ gx, PoolGeom g,
                                                          int chunks)
{
    const int chunk = blockIdx.x % chunks;
    const long long plane = blockIdx.x / chunks;
    const int e = chunk * 256 + threadIdx.x;
    if (e >= g.H * g.W) return;
    const int iy = e / g.W, ix = e - iy * g.W;
    // windows [o*stride, o*stride+size) containing iy / ix
    const int oy_lo = iy < g.size ? 0 : (iy - g.size + g.stride) / g.stride;
    const int oy_hi = min(iy / g.stride, g.OH - 1);
    const int ox_lo = ix < g.size ? 0 : (ix - g.size + g.stride) / g.stride;
    const int ox_hi = min(ix / g.stride, g.OW - 1);
    const long long obase = plane * (long long)g.OH * g.OW;
    const long long flat = plane * (long long)g.H * g.W + e;
    float acc = 0.f;
    for (int oy = oy_lo; oy <= oy_hi; ++oy)
        for (int ox = ox_lo; ox <= ox_hi; ++ox) {
            const long long o = obase + oy * g.OW + ox;
            bool mine;
            if (EXACT) mine = idx_local[o] == e;
            else mine = (long long)argmax[o] == flat;
            if (mine) acc += gy[o];
        }
    gx[flat] = acc;
}

template <bool EXACT>
__global__ __launch_bounds__(256) void maxpool_gradgrad_kernel(const float *__restrict__ ggx,
                                                               const float *__restrict__ argmax,
                                                               const int32_t *__restrict__ idx_local,
                                                               float *__restrict__ ggy,
                                                               long long plane_x, long long plane_y,
                                                               long long total_y)
{
    for (long long o = blockIdx.x * 256LL + threadIdx.x; o < total_y; o += gridDim.x * 256LL) {
        long long src;
        if (EXACT) {
            const int32_t l = idx_local[o];
            src = l >= 0 ? (o / plane_y) * plane_x + l : 0;  // index 0 when nothing beat the start value
        } else {
            src = (long long)argmax[o];
        }
        ggy[o] = ggx[src];
    }
}

static ag_status_t pool_geom(const char *who, int B, int C, int H, int W, int size, int pad,
                             int stride, PoolGeom *g)
{
    AG_REQUIRE(B >= 0 && C >= 0 && H >= 0 && W >= 0, AG_ERR_INVALID_DIMS,
               "%s: negative extent (B=%d C=%d H=%d W=%d)", who, B, C, H, W);
    AG_REQUIRE(size >= 1 && stride >= 1, AG_ERR_INVALID_DIMS, "%s: size and stride must be >= 1 (size=%d stride=%d)",
               who, size, stride);
    AG_REQUIRE(pad == 0, AG_ERR_INVALID_DIMS,
               "%s: pad must be 0 (got %d); the reference's unsigned window start is undefined otherwise",
               who, pad);
    AG_REQUIRE(H >= size && W >= size, AG_ERR_INVALID_DIMS, "%s: window %d larger than the %dx%d plane",
               who, size, H, W);
    AG_REQUIRE((long long)H * W <= 0x7fffffffLL, AG_ERR_INVALID_DIMS, "%s: plane too large", who);
    *g = PoolGeom{H, W, ag_pool_out_size(H, size, pad, stride), ag_pool_out_size(W, size, pad, stride),
                  size, stride};
    return AG_OK;
}

constexpr long long kExactFloatIndexLimit = 1LL << 24;

}  // namespace ag

using namespace ag;

extern "C" ag_status_t ag_maxpool2d_fwd_f32(ag_stream_t stream, const float *x, float *y,
                                            float *argmax, int32_t *idx_local, int B, int C, int H,
                                            int W, int size, int pad, int stride)
{
    PoolGeom g;
    if ((long long)B * C == 0) return AG_OK;
    if (ag_status_t s = pool_geom("max_pool2d", B, C, H, W, size, pad, stride, &g)) return s;
    AG_REQUIRE(x && y && argmax, AG_ERR_INVALID_DIMS, "max_pool2d: null pointer");
    const int chunks = (g.OH * g.OW + 255) / 256;
    const long long blocks = (long long)B * C * chunks;
    AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "max_pool2d: too many tiles (%lld)", blocks);
    hipLaunchKernelGGL(maxpool_fwd_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), x,
                       y, argmax, idx_local, g, chunks);
    return check_launch("max_pool2d");
}

extern "C" ag_status_t ag_maxpool2d_bwd_f32(ag_stream_t stream, const float *gy, const float *argmax,
                                            const int32_t *idx_local, float *gx, int B, int C, int H,
                                            int W, int size, int pad, int stride)
{
    PoolGeom g;
    if ((long long)B * C == 0) return AG_OK;
    if (ag_status_t s = pool_geom("max_pool2d_grad", B, C, H, W, size, pad, stride, &g)) return s;
    AG_REQUIRE(gy && gx && (argmax || idx_local), AG_ERR_INVALID_DIMS, "max_pool2d_grad: null pointer");
    AG_REQUIRE(idx_local || (long long)B * C * H * W <= kExactFloatIndexLimit, AG_ERR_INVALID_DIMS,
               "max_pool2d_grad: an f32 cannot hold offsets into %lld elements exactly (> 2^24); pass the int32 plane-local indices",
               (long long)B * C * H * W);
    const int chunks = (H * W + 255) / 256;
    const long long blocks = (long long)B * C * chunks;
    AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "max_pool2d_grad: too many tiles (%lld)", blocks);
    if (idx_local)
        hipLaunchKernelGGL(maxpool_bwd_kernel<true>, dim3((unsigned)blocks), dim3(256), 0,
                           as_stream(stream), gy, argmax, idx_local, gx, g, chunks);
    else
        hipLaunchKernelGGL(maxpool_bwd_kernel<false>, dim3((unsigned)blocks), dim3(256), 0,
                           as_stream(stream), gy, argmax, idx_local, gx, g, chunks);
    return check_launch("max_pool2d_grad");
}

extern "C" ag_status_t ag_maxpool2d_gradgrad_f32(ag_stream_t stream, const float *ggx,
                                                 const float *argmax, const int32_t *idx_local,
                                                 float *ggy, int B, int C, int H, int W, int size,
                                                 int pad, int stride)
{
    PoolGeom g;
    if ((long long)B * C == 0) return AG_OK;
    if (ag_status_t s = pool_geom("max_pool2d_grad_grad", B, C, H, W, size, pad, stride, &g)) return s;
    AG_REQUIRE(ggx && ggy && (argmax || idx_local), AG_ERR_INVALID_DIMS, "max_pool2d_grad_grad: null pointer");
    AG_REQUIRE(idx_local || (long long)B * C * H * W <= kExactFloatIndexLimit, AG_ERR_INVALID_DIMS,
               "max_pool2d_grad_grad: an f32 cannot hold offsets into %lld elements exactly (> 2^24); pass the int32 plane-local indices",
               (long long)B * C * H * W);
    const long long plane_y = (long long)g.OH * g.OW, total_y = plane_y * B * C;
    if (total_y == 0) return AG_OK;
    long long blocks = (total_y + 255) / 256;
    if (blocks > 262144) blocks = 262144;
    if (idx_local)
        hipLaunchKernelGGL(maxpool_gradgrad_kernel<true>, dim3((unsigned)blocks), dim3(256), 0,
                           as_stream(stream), ggx, argmax, idx_local, ggy, (long long)H * W, plane_y, total_y);
    else
        hipLaunchKernelGGL(maxpool_gradgrad_kernel<false>, dim3((unsigned)blocks), dim3(256), 0,
                           as_stream(stream), ggx, argmax, idx_local, ggy, (long long)H * W, plane_y, total_y);
    return check_launch("max_pool2d_grad_grad");
}
