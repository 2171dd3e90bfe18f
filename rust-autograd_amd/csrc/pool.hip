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

constexpr int kPoolLdsBytes = 32 * 1024;

// LDS-staged forward: one block per (plane, band of R output rows).  The input rows the band
// needs are copied to LDS with coalesced loads (each input byte is fetched once), then every
// thread scans its windows out of LDS.
template <int SIZE, int STRIDE>  // 0 = run-time window / stride
__global__ __launch_bounds__(256) void maxpool_fwd_lds_kernel(const float *__restrict__ x,
                                                              float *__restrict__ y,
                                                              float *__restrict__ argmax,
                                                              int32_t *__restrict__ idx_local,
                                                              PoolGeom g, int R, int bands, int vec)
{
    extern __shared__ float tile[];
    const int size = SIZE ? SIZE : g.size, stride = STRIDE ? STRIDE : g.stride;
    const int band = blockIdx.x % bands;
    const long long plane = blockIdx.x / bands;
    const int oy0 = band * R;
    const int rows = min(R, g.OH - oy0);
    const int iy0 = oy0 * stride;
    const int in_rows = (rows - 1) * stride + size;
    const long long base = plane * (long long)g.H * g.W;
    const float *xp = x + base + (long long)iy0 * g.W;
    const int n_in = in_rows * g.W;
    if (vec) {
        const float4 *x4 = reinterpret_cast<const float4 *>(xp);
        float4 *t4 = reinterpret_cast<float4 *>(tile);
        for (int e = threadIdx.x; e < n_in / 4; e += 256) t4[e] = ld_stream(x4 + e);
    } else {
        for (int e = threadIdx.x; e < n_in; e += 256) tile[e] = xp[e];
    }
    __syncthreads();
    const long long obase = plane * (long long)g.OH * g.OW + (long long)oy0 * g.OW;
    for (int o = threadIdx.x; o < rows * g.OW; o += 256) {
        const int r = o / g.OW, ox = o - r * g.OW;
        const float *w0 = tile + (r * stride) * g.W + ox * stride;
        float best = -FLT_MAX;
        int best_local = -1;
#pragma unroll
        for (int dy = 0; dy < size; ++dy)
#pragma unroll
            for (int dx = 0; dx < size; ++dx) {
                const float v = w0[dy * g.W + dx];
                if (v > best) {
                    best = v;
                    best_local = (iy0 + r * stride + dy) * g.W + ox * stride + dx;
                }
            }
        st_stream(y + obase + o, best);
        const unsigned long long flat = best_local >= 0 ? (unsigned long long)(base + best_local) : 0ull;
        st_stream(argmax + obase + o, (float)flat);
        if (idx_local) st_stream(idx_local + obase + o, best_local);
    }
}

// LDS-staged backward: one block per (plane, band of IR input rows).  The upstream gradient and
// the selection indices of every window that can touch the band are staged in LDS; each thread
// then produces four consecutive pixels (one 128-bit store), visiting candidate windows in
// ascending (oy, ox) order.
template <bool EXACT, int SIZE, int STRIDE>  // SIZE/STRIDE 0 = run-time
__global__ __launch_bounds__(256) void maxpool_bwd_lds_kernel(const float *__restrict__ gy,
                                                              const float *__restrict__ argmax,
                                                              const int32_t *__restrict__ idx_local,
                                                              float *__restrict__ gx, PoolGeom g,
                                                              int IR, int bands, int max_orows)
{
    extern __shared__ float smem[];
    float *s_gy = smem;
    int *s_idx = reinterpret_cast<int *>(smem + max_orows * g.OW);
    const int size = SIZE ? SIZE : g.size, stride = STRIDE ? STRIDE : g.stride;
    const int band = blockIdx.x % bands;
    const long long plane = blockIdx.x / bands;
    const int iy0 = band * IR;
    const int rows = min(IR, g.H - iy0);
    const int iy1 = iy0 + rows - 1;
    // output rows whose window intersects [iy0, iy1]
    const int o_lo = iy0 < size ? 0 : (iy0 - size + stride) / stride;
    const int o_hi = min(iy1 / stride, g.OH - 1);
    const int n_o = max(0, o_hi - o_lo + 1) * g.OW;
    const long long obase = plane * (long long)g.OH * g.OW + (long long)o_lo * g.OW;
    const long long xbase = plane * (long long)g.H * g.W;
    for (int e = threadIdx.x; e < n_o; e += 256) {
        s_gy[e] = ld_stream(gy + obase + e);
        if (EXACT) {
            s_idx[e] = ld_stream(idx_local + obase + e);
        } else {
            // whole-tensor offset -> plane-local (exact below 2^24 elements); other planes never match
            const long long a = (long long)argmax[obase + e] - xbase;
            s_idx[e] = (a >= 0 && a < (long long)g.H * g.W) ? (int)a : -1;
        }
    }
    __syncthreads();
    // A pixel lies in at most CAND windows per axis; they are visited in ascending order.
    constexpr int CAND = (SIZE && STRIDE) ? (SIZE + STRIDE - 1) / STRIDE : 0;
    const int W4 = g.W >> 2;
    for (int q = threadIdx.x; q < rows * W4; q += 256) {
        const int r = q / W4, ix0 = (q - r * W4) * 4;
        const int iy = iy0 + r;
        const int oy_lo = iy < size ? 0 : (iy - size + stride) / stride;
        const int oy_hi = min(iy / stride, g.OH - 1);
        float out[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int ix = ix0 + k;
            const int ox_lo = ix < size ? 0 : (ix - size + stride) / stride;
            const int ox_hi = min(ix / stride, g.OW - 1);
            const int me = iy * g.W + ix;
            float acc = 0.f;
            if (CAND) {
#pragma unroll
                for (int a = CAND - 1; a >= 0; --a) {
                    const int oy = iy / stride - a;
                    if (oy < oy_lo || oy > oy_hi) continue;
#pragma unroll
                    for (int b = CAND - 1; b >= 0; --b) {
                        const int ox = ix / stride - b;
                        if (ox < ox_lo || ox > ox_hi) continue;
                        const int o = (oy - o_lo) * g.OW + ox;
                        if (s_idx[o] == me) acc += s_gy[o];
                    }
                }
            } else {
                for (int oy = oy_lo; oy <= oy_hi; ++oy)
                    for (int ox = ox_lo; ox <= ox_hi; ++ox) {
                        const int o = (oy - o_lo) * g.OW + ox;
                        if (s_idx[o] == me) acc += s_gy[o];
                    }
            }
            out[k] = acc;
        }
        st_stream(reinterpret_cast<float4 *>(gx + xbase + (long long)iy * g.W + ix0),
                  make_float4(out[0], out[1], out[2], out[3]));
    }
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
    if (g.OH <= 0 || g.OW <= 0) return AG_OK;
    const long long row_bytes = (long long)W * 4;
    if (row_bytes * size <= kPoolLdsBytes) {
        // rows of output per band so that the staged input rows fit the LDS budget
        int R = (int)((kPoolLdsBytes / row_bytes - size) / stride + 1);
        if (R > g.OH) R = g.OH;
        const int bands = (g.OH + R - 1) / R;
        const long long blocks = (long long)B * C * bands;
        AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "max_pool2d: too many tiles (%lld)", blocks);
        const size_t lds = (size_t)((R - 1) * stride + size) * row_bytes;
        const int vec = (W % 4 == 0) && aligned16(x);
#define AG_POOL_FWD(SZ, ST)                                                                                   \
    hipLaunchKernelGGL((maxpool_fwd_lds_kernel<SZ, ST>), dim3((unsigned)blocks), dim3(256), lds, as_stream(stream), \
                       x, y, argmax, idx_local, g, R, bands, vec)
        if (size == 3 && stride == 2) AG_POOL_FWD(3, 2);
        else if (size == 2 && stride == 2) AG_POOL_FWD(2, 2);
        else AG_POOL_FWD(0, 0);
#undef AG_POOL_FWD
    } else {
        const int chunks = (g.OH * g.OW + 255) / 256;
        const long long blocks = (long long)B * C * chunks;
        AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "max_pool2d: too many tiles (%lld)", blocks);
        hipLaunchKernelGGL(maxpool_fwd_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), x, y,
                           argmax, idx_local, g, chunks);
    }
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
    // LDS-staged path: W % 4 == 0 (128-bit stores) and the windows of a band fit the budget
    const long long orow_bytes = (long long)g.OW * 8;  // gy + index per output
    if (W % 4 == 0 && aligned16(gx) && g.OH > 0 && g.OW > 0 &&
        orow_bytes * ((size + stride - 1) / stride + 1) <= kPoolLdsBytes) {
        // IR input rows touch at most IR/stride + size/stride + 2 output rows
        const int budget_rows = (int)(kPoolLdsBytes / orow_bytes);
        int IR = (budget_rows - (size + stride - 1) / stride - 2) * stride;
        if (IR < 1) IR = 1;
        if (IR > H) IR = H;
        const int bands = (H + IR - 1) / IR;
        int max_orows = (IR - 1) / stride + (size + stride - 1) / stride + 2;
        if (max_orows > g.OH) max_orows = g.OH;
        const long long blocks = (long long)B * C * bands;
        AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "max_pool2d_grad: too many tiles (%lld)", blocks);
        const size_t lds = (size_t)max_orows * orow_bytes;
#define AG_POOL_BWD(EX, SZ, ST)                                                                               \
    hipLaunchKernelGGL((maxpool_bwd_lds_kernel<EX, SZ, ST>), dim3((unsigned)blocks), dim3(256), lds,               \
                       as_stream(stream), gy, argmax, idx_local, gx, g, IR, bands, max_orows)
        const bool s32 = size == 3 && stride == 2, s22 = size == 2 && stride == 2;
        if (idx_local) {
            if (s32) AG_POOL_BWD(true, 3, 2);
            else if (s22) AG_POOL_BWD(true, 2, 2);
            else AG_POOL_BWD(true, 0, 0);
        } else {
            if (s32) AG_POOL_BWD(false, 3, 2);
            else if (s22) AG_POOL_BWD(false, 2, 2);
            else AG_POOL_BWD(false, 0, 0);
        }
#undef AG_POOL_BWD
        return check_launch("max_pool2d_grad");
    }
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
