// MaxPool2D forward, argmax backward and the argmax gather used by the second-order op.
//
// All three are HBM-bound elementwise-style kernels over NCHW planes.  The backward is written
// as a gather: each input pixel visits the (few) windows that contain it in ascending (oy, ox)
// order and adds the upstream gradient of those that selected it.  That is the order in which
// the reference's sequential scatter `gx[argmax[i]] += gy[i]` (max_pool2d.rs:123-131) reaches the
// pixel, so sums are bit-identical and no atomics or zero-fill pass are needed.
#include <cfloat>

#include "ag_internal.h"
#ifdef AG_TEST_HOOKS
#include "ag_test_hooks.h"
#endif

namespace ag {

struct PoolGeom {
    int H, W, OH, OW, size, stride;
};

// The exact selection of a window travels as ONE BYTE per output: the tap dy*size + dx of the first
// strict maximum inside the window (row-major, the reference's scan order), kNoTap when no element
// exceeded the start value (an all-NaN window).  The backward knows the window geometry, so the
// byte identifies the pixel; it replaces the reference's f32-encoded whole-tensor offset, which is
// exact only up to 2^24 elements, at a quarter of the bytes.
constexpr int kNoTap = 255;
constexpr int kMaxTapSize = 15;  // size*size - 1 must stay below kNoTap

// Plane-local position of the pixel that window (oy, ox) selected, -1 for kNoTap.
__device__ inline int tap_position(int tap, int oy, int ox, const PoolGeom &g)
{
    if (tap == kNoTap) return -1;
    const int dy = tap / g.size, dx = tap - dy * g.size;
    return (oy * g.stride + dy) * g.W + ox * g.stride + dx;
}

__global__ __launch_bounds__(256) void maxpool_fwd_kernel(const float *__restrict__ x,
                                                          float *__restrict__ y,
                                                          float *__restrict__ argmax,
                                                          uint8_t *__restrict__ taps,
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
    int best_local = -1, best_tap = kNoTap;
    for (int h = h0; h < h1; ++h)
        for (int w = w0; w < w1; ++w) {
            const float v = xp[h * g.W + w];
            if (v > best) {
                best = v;
                best_local = h * g.W + w;
                best_tap = (h - h0) * g.size + (w - w0);
            }
        }
    const long long out = plane * (long long)g.OH * g.OW + o;
    y[out] = best;
    // The reference stores the whole-tensor offset converted to f32 by value (max_pool2d.rs:74-75).
    const unsigned long long flat = best_local >= 0 ? (unsigned long long)(base + best_local) : 0ull;
    argmax[out] = (float)flat;  // round-to-nearest-even, like Rust's `as f32`
    if (taps) taps[out] = (uint8_t)best_tap;
}

// The factor of a ReLU's gradient (activation_ops.rs:161-166: greater(x, 0) * gy) that the backward kernels apply
// to what they store when they are given the ReLU's input or output as `relu_x` (null = none).
__device__ inline float relu_gate(float v) { return v > 0.f ? 1.f : 0.f; }

// EXACT: selection read from the tap bytes; otherwise from the f32 argmax.
template <bool EXACT, bool RELU>
__global__ __launch_bounds__(256) void maxpool_bwd_kernel(const float *__restrict__ gy,
                                                          const float *__restrict__ argmax,
                                                          const uint8_t *__restrict__ taps,
                                                          const float *__restrict__ relu_x,
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
            if (EXACT) mine = tap_position(taps[o], oy, ox, g) == e;
            else mine = (long long)argmax[o] == flat;
            if (mine) acc += gy[o];
        }
    gx[flat] = RELU ? relu_gate(relu_x[flat]) * acc : acc;
}

// 2 x 2 windows at stride 2 over a plane with even extents: the windows tile the plane, so every input
// pixel belongs to exactly one window and each thread writes the four pixels of its own window
// (two 8-byte stores; a wave's stores cover two whole input rows of contiguous memory).
template <bool EXACT, bool RELU>
__global__ __launch_bounds__(256) void maxpool_bwd_tile2_kernel(const float *__restrict__ gy,
                                                                const float *__restrict__ argmax,
                                                                const uint8_t *__restrict__ taps,
                                                                const float *__restrict__ relu_x,
                                                                float *__restrict__ gx, PoolGeom g,
                                                                long long outputs)
{
    const long long o = blockIdx.x * 256ll + threadIdx.x;
    if (o >= outputs) return;
    const int per_plane = g.OH * g.OW;
    const long long plane = o / per_plane;
    const int e = (int)(o - plane * per_plane);
    const int oy = e / g.OW, ox = e - oy * g.OW;
    const long long xbase = plane * (long long)g.H * g.W;
    int tap;  // 0..3 = dy * 2 + dx, anything else = none
    if (EXACT) {
        tap = taps[o];
    } else {
        // whole-tensor offset -> tap inside this window (exact below 2^24 elements)
        const long long a = (long long)argmax[o] - xbase - (long long)(2 * oy) * g.W - 2 * ox;
        tap = a == 0 ? 0 : a == 1 ? 1 : a == g.W ? 2 : a == g.W + 1 ? 3 : kNoTap;
    }
    // 0 + gy as in the reference's scatter onto a zeroed plane (max_pool2d.rs:123-131) and in the gather kernels:
    // a gradient of -0.0 (what an upstream 0 * negative leaves) arrives as +0.0
    const float v = 0.f + gy[o];
    float2 top, bottom;
    top.x = tap == 0 ? v : 0.f;
    top.y = tap == 1 ? v : 0.f;
    bottom.x = tap == 2 ? v : 0.f;
    bottom.y = tap == 3 ? v : 0.f;
    const long long at = xbase + (long long)(2 * oy) * g.W + 2 * ox;
    if (RELU) {
        const float2 mt = *reinterpret_cast<const float2 *>(relu_x + at), mb = *reinterpret_cast<const float2 *>(relu_x + at + g.W);
        top.x = relu_gate(mt.x) * top.x;
        top.y = relu_gate(mt.y) * top.y;
        bottom.x = relu_gate(mb.x) * bottom.x;
        bottom.y = relu_gate(mb.y) * bottom.y;
    }
    float *row = gx + at;
    *reinterpret_cast<float2 *>(row) = top;
    *reinterpret_cast<float2 *>(row + g.W) = bottom;
}

// Forward of 2 x 2 windows at stride 2 over a plane with even extents, one thread per window: two 8-byte loads (a
// wave's loads cover two whole input rows of contiguous memory), the scan in the reference's order (first maximum
// wins, strict comparison starting from -FLT_MAX), three coalesced stores.  No staging and no barrier: on the small
// planes of a launch-bound network ([128,32,28,28]: 8.2 -> about 5 us) that is what the time went to.  Large tensors
// with rows of whole quads stay on the staged kernel.
__global__ __launch_bounds__(256) void maxpool_fwd_tile2_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                float *__restrict__ argmax, uint8_t *__restrict__ taps,
                                                                PoolGeom g, long long outputs)
{
    const long long o = blockIdx.x * 256ll + threadIdx.x;
    if (o >= outputs) return;
    const int per_plane = g.OH * g.OW;
    const long long plane = o / per_plane;
    const int e = (int)(o - plane * per_plane);
    const int oy = e / g.OW, ox = e - oy * g.OW;
    const long long at = plane * (long long)g.H * g.W + (long long)(2 * oy) * g.W + 2 * ox;  // whole-tensor offset of tap 0
    const float2 top = *reinterpret_cast<const float2 *>(x + at), bottom = *reinterpret_cast<const float2 *>(x + at + g.W);
    const float v[4] = {top.x, top.y, bottom.x, bottom.y};
    float best = -FLT_MAX;
    int best_tap = kNoTap;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const bool gt = v[t] > best;
        best = gt ? v[t] : best;
        best_tap = gt ? t : best_tap;
    }
    const long long flat = at + (best_tap >> 1) * g.W + (best_tap & 1);
    y[o] = best;
    argmax[o] = best_tap != kNoTap ? (float)(unsigned long long)flat : 0.f;  // the offset by value, rounded to nearest even
    if (taps) taps[o] = (uint8_t)best_tap;
}

// The activation in front of such a pooling in the same pass: r = relu(a + b) (b broadcast along the axes where its
// extent is 1; null = relu(a)) is written out -- the backward needs it -- and pooled as it is produced.  One
// thread per window as above; the sum is rounded to f32 before the maximum and the maximum before the comparison,
// so r, y, argmax and the tap bytes have the bits of the separate kernels.
struct BiasStrides {
    long long n, c, h, w;  // element strides of b along the axes of a (0 where b is broadcast)
};
__global__ __launch_bounds__(256) void relu_maxpool_tile2_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                                 BiasStrides bs, float *__restrict__ r, float *__restrict__ y,
                                                                 float *__restrict__ argmax, uint8_t *__restrict__ taps,
                                                                 PoolGeom g, int C, long long outputs)
{
    const long long o = blockIdx.x * 256ll + threadIdx.x;
    if (o >= outputs) return;
    const int per_plane = g.OH * g.OW;
    const long long plane = o / per_plane;
    const int e = (int)(o - plane * per_plane);
    const int oy = e / g.OW, ox = e - oy * g.OW;
    const long long at = plane * (long long)g.H * g.W + (long long)(2 * oy) * g.W + 2 * ox;  // whole-tensor offset of tap 0
    const float2 top = *reinterpret_cast<const float2 *>(a + at), bottom = *reinterpret_cast<const float2 *>(a + at + g.W);
    float v[4] = {top.x, top.y, bottom.x, bottom.y};
    if (b) {
        const long long n = plane / C;
        const int c = (int)(plane - n * C);
        const float *bp = b + n * bs.n + c * bs.c + (long long)(2 * oy) * bs.h + (long long)(2 * ox) * bs.w;
        v[0] = v[0] + bp[0];
        v[1] = v[1] + bp[bs.w];
        v[2] = v[2] + bp[bs.h];
        v[3] = v[3] + bp[bs.h + bs.w];
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) v[t] = v[t] > 0.f ? v[t] : 0.f;  // activation_ops.rs:155-159 (a NaN becomes 0)
    *reinterpret_cast<float2 *>(r + at) = make_float2(v[0], v[1]);
    *reinterpret_cast<float2 *>(r + at + g.W) = make_float2(v[2], v[3]);
    float best = -FLT_MAX;
    int best_tap = kNoTap;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const bool gt = v[t] > best;
        best = gt ? v[t] : best;
        best_tap = gt ? t : best_tap;
    }
    const long long flat = at + (best_tap >> 1) * g.W + (best_tap & 1);
    y[o] = best;
    argmax[o] = best_tap != kNoTap ? (float)(unsigned long long)flat : 0.f;
    if (taps) taps[o] = (uint8_t)best_tap;
}

constexpr int kPoolLdsBytes = 32 * 1024;
// A plane that does not fit half of that is cut into bands of at most this many staged bytes:
// eight resident blocks per CU measured better than fewer, larger ones (112x112 planes: 0.242 ms
// against 0.286 ms), while planes that fit are best taken whole.
constexpr int kPoolBandBytes = 8 * 1024;

// Scans the windows of `rows` output rows (starting at output row oy0 of plane `plane`) out of the
// staged input rows in `tile` (row pitch W, first staged row = input row iy0) and writes the three
// outputs.  256 threads, 256 outputs per round.
template <int SIZE, int STRIDE>  // 0 = run-time window / stride
__device__ inline void pool_scan_band(const float *tile, float *__restrict__ y, float *__restrict__ argmax,
                                      uint8_t *__restrict__ taps, const PoolGeom &g, long long plane,
                                      int oy0, int rows, int iy0)
{
    const int size = SIZE ? SIZE : g.size, stride = STRIDE ? STRIDE : g.stride;
    const long long base = plane * (long long)g.H * g.W;
    const long long obase = plane * (long long)g.OH * g.OW + (long long)oy0 * g.OW;
    float *const yp = y + obase;
    float *const ap = argmax + obase;
    uint8_t *const tp = taps ? taps + obase : nullptr;
    // whole-tensor offsets below 2^32 convert to f32 with one instruction
    const bool small = (unsigned long long)(base + (long long)g.H * g.W) <= 0xffffffffull;
    const int OW = g.OW, W = g.W, n_out = rows * OW;
    // (r, ox) of output o, advanced by 256 outputs per round without a division
    const int step_r = 256 / OW, step_x = 256 - step_r * OW;
    int r = threadIdx.x / OW, ox = threadIdx.x - r * OW;
    for (int o = threadIdx.x; o < n_out; o += 256) {
        const int first = (r * stride) * W + ox * stride;  // window's first element inside the staged rows
        const float *w0 = tile + first;
        float best = -FLT_MAX;
        int best_off = -1, best_tap = kNoTap;
#pragma unroll
        for (int dy = 0; dy < size; ++dy)
#pragma unroll
            for (int dx = 0; dx < size; ++dx) {
                const float v = w0[dy * W + dx];
                const bool gt = v > best;
                best = gt ? v : best;
                best_off = gt ? dy * W + dx : best_off;
                best_tap = gt ? dy * size + dx : best_tap;
            }
        const int best_local = best_off >= 0 ? iy0 * W + first + best_off : -1;
        float flat;
        if (small) flat = best_off >= 0 ? (float)((unsigned)base + (unsigned)best_local) : 0.f;
        else flat = best_off >= 0 ? (float)(unsigned long long)(base + best_local) : 0.f;
        st_stream(yp + o, best);
        st_stream(ap + o, flat);
        if (tp) tp[o] = (uint8_t)best_tap;
        r += step_r;
        ox += step_x;
        if (ox >= OW) {
            ox -= OW;
            ++r;
        }
    }
}

// LDS-staged forward: one block per (plane, band of R output rows).  The input rows the band
// needs are copied to LDS with coalesced loads (each input byte is fetched once), then every
// thread scans its windows out of LDS.
template <int SIZE, int STRIDE>  // 0 = run-time window / stride
__global__ __launch_bounds__(256) void maxpool_fwd_lds_kernel(const float *__restrict__ x,
                                                              float *__restrict__ y,
                                                              float *__restrict__ argmax,
                                                              uint8_t *__restrict__ taps,
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
        // Four loads are in flight per thread before the first LDS write.  Written as a plain copy loop
        // the compiler waits for every load before it issues the next, and a block pays the memory
        // latency once per 4 KB instead of once per 16 KB (measured: 0.1135 -> 0.108 ms on the
        // [256,128,56,56] 3x3 stride-2 case, whose planes take three loads per thread).
        const float4 *x4 = reinterpret_cast<const float4 *>(xp);
        float4 *t4 = reinterpret_cast<float4 *>(tile);
        const int n4 = n_in / 4;
        for (int e0 = 0; e0 < n4; e0 += 1024) {
            float4 v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int e = e0 + j * 256 + threadIdx.x;
                if (e < n4) v[j] = ld_stream(x4 + e);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int e = e0 + j * 256 + threadIdx.x;
                if (e < n4) t4[e] = v[j];
            }
        }
    } else {
        for (int e = threadIdx.x; e < n_in; e += 256) tile[e] = xp[e];
    }
    __syncthreads();
    pool_scan_band<SIZE, STRIDE>(tile, y, argmax, taps, g, plane, oy0, rows, iy0);
}

// LDS-staged backward: one block per (plane, band of IR input rows).  The upstream gradient and
// the selection indices of every window that can touch the band are staged in LDS; each thread
// then produces four consecutive pixels (one 128-bit store), visiting candidate windows in
// ascending (oy, ox) order.
template <bool EXACT, int SIZE, int STRIDE, bool RELU>  // SIZE/STRIDE 0 = run-time
__global__ __launch_bounds__(256) void maxpool_bwd_lds_kernel(const float *__restrict__ gy,
                                                              const float *__restrict__ argmax,
                                                              const uint8_t *__restrict__ taps,
                                                              const float *__restrict__ relu_x,
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
            const int orow = e / g.OW;
            s_idx[e] = tap_position(taps[obase + e], o_lo + orow, e - orow * g.OW, g);
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
        const long long at = xbase + (long long)iy * g.W + ix0;
        if (RELU) {
            const float4 m = ld_stream(reinterpret_cast<const float4 *>(relu_x + at));
            out[0] = relu_gate(m.x) * out[0];
            out[1] = relu_gate(m.y) * out[1];
            out[2] = relu_gate(m.z) * out[2];
            out[3] = relu_gate(m.w) * out[3];
        }
        st_stream(reinterpret_cast<float4 *>(gx + at), make_float4(out[0], out[1], out[2], out[3]));
    }
}

template <bool EXACT>
__global__ __launch_bounds__(256) void maxpool_gradgrad_kernel(const float *__restrict__ ggx,
                                                               const float *__restrict__ argmax,
                                                               const uint8_t *__restrict__ taps,
                                                               float *__restrict__ ggy, PoolGeom g,
                                                               long long plane_x, long long plane_y,
                                                               long long total_y)
{
    for (long long o = blockIdx.x * 256LL + threadIdx.x; o < total_y; o += gridDim.x * 256LL) {
        long long src;
        if (EXACT) {
            const long long plane = o / plane_y;
            const int in_plane = (int)(o - plane * plane_y), oy = in_plane / g.OW;
            const int l = tap_position(taps[o], oy, in_plane - oy * g.OW, g);
            src = l >= 0 ? plane * plane_x + l : 0;  // index 0 when nothing beat the start value
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

// ---------------------------------------------------------------------------------------------
// Stride-2 backward without LDS (window 2 or 3, W % 4 == 0, W <= 256).  LPR lanes (a power of
// two >= W/4) share one plane; lane q owns input columns 4q .. 4q+3 and reads the two outputs 2q
// and 2q+1 whose windows start there.  A lane walks a chunk of output rows top to bottom and
// writes every input row once with an aligned 128-bit streaming store.
// ---------------------------------------------------------------------------------------------
// A chunk of output rows [oy0, oy1) owns the input rows
// [2*oy0, 2*oy1) (the last chunk also the rows below the last window, which receive nothing).
// Every pixel adds the gradients of the windows that selected it in ascending (oy, ox) order,
// the order of the reference's scatter loop, so the sums are bit-identical.  For the 3-wide
// window the contributions of window row oy to input row 2*oy+2 are carried to the next
// iteration, and a chunk first recomputes what the window row above it contributes to its top row.
template <bool EXACT, int SIZE, int LPR, bool RELU>
__global__ __launch_bounds__(256) void maxpool_bwd_s2_kernel(const float *__restrict__ gy,
                                                             const float *__restrict__ argmax,
                                                             const uint8_t *__restrict__ taps,
                                                             const float *__restrict__ relu_x,
                                                             float *__restrict__ gx, PoolGeom g, int rows_per_chunk,
                                                             int chunks, unsigned groups_total)
{
    constexpr int GPW = 64 / LPR;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int q = lane & (LPR - 1);
    const bool in_row = q < (g.W >> 2);
    const int W = g.W;
    for (unsigned grp = (blockIdx.x * 4u + wave) * GPW + lane / LPR; grp - lane / LPR < groups_total;
         grp += gridDim.x * 4u * GPW) {
        const bool active = in_row && grp < groups_total;
        const unsigned plane = grp / (unsigned)chunks;
        const int chunk = (int)(grp - plane * (unsigned)chunks);
        const int oy0 = chunk * rows_per_chunk;
        const int oy1 = grp < groups_total ? min(oy0 + rows_per_chunk, g.OH) : oy0;
        const bool last_chunk = chunk == chunks - 1;
        const long long base = (long long)plane * g.H * W;
        const long long obase = (long long)plane * g.OH * g.OW;
        float *gxp = gx + base + q * 4;
        const bool va = active && 2 * q < g.OW, vb = active && 2 * q + 1 < g.OW;
        // gradient and selected plane-local position of outputs (oy, 2q) and (oy, 2q+1)
        struct Out {
            float ga, gb;
            int ia, ib;
        };
        auto load_out = [&](int oy) {
            Out o;
            const long long at = obase + (long long)oy * g.OW + 2 * q;
            o.ga = va ? gy[at] : 0.f;
            o.gb = vb ? gy[at + 1] : 0.f;
            if (EXACT) {
                // tap -> pixel: window (oy, ox) starts at (2*oy, 2*ox).  (Plain loads: a cache line of
                // gradients or taps serves several consecutive rows of the walk.)
                const int ta = va ? (int)taps[at] : kNoTap, tb = vb ? (int)taps[at + 1] : kNoTap;
                o.ia = ta != kNoTap ? (2 * oy + ta / SIZE) * W + 4 * q + ta % SIZE : -1;
                o.ib = tb != kNoTap ? (2 * oy + tb / SIZE) * W + 4 * q + 2 + tb % SIZE : -1;
            } else {
                // whole-tensor offsets as stored by the forward pass; made plane-local here
                const long long hw = (long long)g.H * W;
                const long long da = va ? (long long)argmax[at] - base : -1, db = vb ? (long long)argmax[at + 1] - base : -1;
                o.ia = da >= 0 && da < hw ? (int)da : -1;
                o.ib = db >= 0 && db < hw ? (int)db : -1;
            }
            return o;
        };
        // Adds what window row `o` (with the neighbour's second window `pg`, `pi`) gives to the
        // four pixels of input row iy, pixel by pixel in ascending ox.
        auto add_row = [&](float (&acc)[4], const Out &o, float pg, int pi, int iy) {
            const int r = iy * W + 4 * q;
            if (SIZE == 3) {
                acc[0] = pi == r ? acc[0] + pg : acc[0];
                acc[0] = o.ia == r ? acc[0] + o.ga : acc[0];
                acc[1] = o.ia == r + 1 ? acc[1] + o.ga : acc[1];
                acc[2] = o.ia == r + 2 ? acc[2] + o.ga : acc[2];
                acc[2] = o.ib == r + 2 ? acc[2] + o.gb : acc[2];
                acc[3] = o.ib == r + 3 ? acc[3] + o.gb : acc[3];
            } else {
                acc[0] = o.ia == r ? acc[0] + o.ga : acc[0];
                acc[1] = o.ia == r + 1 ? acc[1] + o.ga : acc[1];
                acc[2] = o.ib == r + 2 ? acc[2] + o.gb : acc[2];
                acc[3] = o.ib == r + 3 ? acc[3] + o.gb : acc[3];
            }
        };
        auto neighbour = [&](const Out &o, float &pg, int &pi) {
            pg = __shfl_up(o.gb, 1, LPR);
            pi = __shfl_up(o.ib, 1, LPR);
            if (q == 0) {
                pg = 0.f;
                pi = -1;
            }
        };
        // the ReLU's values at the four pixels of input row iy (loaded ahead of the sums they will gate)
        auto load_mask = [&](int iy) {
            return RELU && active ? ld_stream(reinterpret_cast<const float4 *>(relu_x + base + q * 4 + iy * W))
                                  : make_float4(1.f, 1.f, 1.f, 1.f);
        };
        auto store_row = [&](int iy, const float (&acc)[4], const float4 &m) {
            if (!active) return;
            float4 v = make_float4(acc[0], acc[1], acc[2], acc[3]);
            if (RELU) v = make_float4(relu_gate(m.x) * v.x, relu_gate(m.y) * v.y, relu_gate(m.z) * v.z, relu_gate(m.w) * v.w);
            st_stream(reinterpret_cast<float4 *>(gxp + iy * W), v);
        };
        float carry[4] = {0.f, 0.f, 0.f, 0.f};
        Out cur;
        cur.ga = cur.gb = 0.f;
        cur.ia = cur.ib = -1;
        if (SIZE == 3 && oy0 > 0 && oy0 < oy1) {
            const Out above = load_out(oy0 - 1);
            float pg;
            int pi;
            neighbour(above, pg, pi);
            add_row(carry, above, pg, pi, 2 * oy0);
        }
        if (oy0 < oy1) cur = load_out(oy0);
        for (int oy = oy0; oy < oy1; ++oy) {
            Out nxt;
            nxt.ga = nxt.gb = 0.f;
            nxt.ia = nxt.ib = -1;
            if (oy + 1 < oy1) nxt = load_out(oy + 1);
            const float4 m0 = load_mask(2 * oy), m1 = load_mask(2 * oy + 1);
            float pg = 0.f;
            int pi = -1;
            if (SIZE == 3) neighbour(cur, pg, pi);
            float a0[4] = {carry[0], carry[1], carry[2], carry[3]}, a1[4] = {0.f, 0.f, 0.f, 0.f};
            add_row(a0, cur, pg, pi, 2 * oy);
            add_row(a1, cur, pg, pi, 2 * oy + 1);
            store_row(2 * oy, a0, m0);
            store_row(2 * oy + 1, a1, m1);
            if (SIZE == 3) {
                carry[0] = carry[1] = carry[2] = carry[3] = 0.f;
                add_row(carry, cur, pg, pi, 2 * oy + 2);
            }
            cur = nxt;
        }
        if (last_chunk && grp < groups_total) {
            // rows below the last window row: the carried row (3-wide window), then zeros
            int iy = 2 * g.OH;
            if (SIZE == 3 && iy < g.H) {
                store_row(iy, carry, load_mask(iy));
                ++iy;
            }
            const float z[4] = {0.f, 0.f, 0.f, 0.f};
            for (; iy < g.H; ++iy) store_row(iy, z, load_mask(iy));
        }
    }
}

static int lanes_per_row(int W)
{
    const int W4 = W >> 2;
    return W4 <= 4 ? 4 : W4 <= 8 ? 8 : W4 <= 16 ? 16 : W4 <= 32 ? 32 : 64;
}

#ifdef AG_TEST_HOOKS
static thread_local int g_chunk_rows = 0;  // test hook (ag_test_hooks.h; test flavour of the library only), per calling thread
#else
constexpr int g_chunk_rows = 0;
#endif
// Output rows per chunk of the stride-2 backward.  Short chunks win by a wide margin although each
// re-reads the window row above it (one byte and one float per output): 256 x 128 planes of
// 56 x 56 take 0.120 ms as whole planes, 0.113 with 9 rows, 0.103 with 3 and 0.082-0.091 with 2
// (one row: 0.096-0.114).
static int pool_chunk_rows(int OH)
{
    if (g_chunk_rows > 0) return g_chunk_rows < OH ? g_chunk_rows : OH;
    return OH < 2 ? OH : 2;
}

constexpr long long kExactFloatIndexLimit = 1LL << 24;

}  // namespace ag

using namespace ag;

#ifdef AG_TEST_HOOKS
// Test hook (ag_test_hooks.h; not part of the operator surface and not in the shipped library): output rows per
// chunk of the stride-2 pooling kernels for later calls of this thread (0 = automatic; negative: automatic, and
// 2 x 2 windows stay off the one-thread-per-window kernels where another kernel can take them).
extern "C" void ag_test_pool_chunk_rows(int rows) { ag::g_chunk_rows = rows; }
#endif

extern "C" ag_status_t ag_maxpool2d_fwd_f32(ag_stream_t stream, const float *x, float *y,
                                            float *argmax, uint8_t *taps, int B, int C, int H,
                                            int W, int size, int pad, int stride)
{
    PoolGeom g;
    if ((long long)B * C == 0) return AG_OK;
    if (ag_status_t s = pool_geom("max_pool2d", B, C, H, W, size, pad, stride, &g)) return s;
    AG_REQUIRE(x && y && argmax, AG_ERR_INVALID_DIMS, "max_pool2d: null pointer");
    AG_REQUIRE(!taps || size <= kMaxTapSize, AG_ERR_INVALID_DIMS,
               "max_pool2d: a tap byte addresses windows of up to %d x %d (got %d)", kMaxTapSize, kMaxTapSize, size);
    if (g.OH <= 0 || g.OW <= 0) return AG_OK;
    const long long row_bytes = (long long)W * 4;
    // (up to 2^23 elements, where a launch's set-up counts, and for rows that are no whole quads; beyond that the
    // staged kernel's 16-byte loads win: [256,128,112,112] 0.41 against 0.44 ms)
    const bool tile2 = W % 4 != 0 || ((long long)B * C * H * W <= (1LL << 23) && g_chunk_rows >= 0);
    if (size == 2 && stride == 2 && H % 2 == 0 && W % 2 == 0 && ((uintptr_t)x & 7u) == 0 && tile2) {
        const long long outputs = (long long)B * C * g.OH * g.OW, blocks = (outputs + 255) / 256;
        AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "max_pool2d: too many tiles (%lld)", blocks);
        hipLaunchKernelGGL(maxpool_fwd_tile2_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), x, y, argmax,
                           taps, g, outputs);
    } else if (row_bytes * size <= kPoolLdsBytes) {
        // rows of output per band so that the staged input rows fit the LDS budget
        const long long budget = (long long)H * row_bytes <= kPoolLdsBytes / 2 || row_bytes * size > kPoolBandBytes
                                     ? kPoolLdsBytes : kPoolBandBytes;
        int R = (int)((budget / row_bytes - size) / stride + 1);
        if (R > g.OH) R = g.OH;
        const int bands = (g.OH + R - 1) / R;
        R = (g.OH + bands - 1) / bands;  // bands of equal height
        const long long blocks = (long long)B * C * bands;
        AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "max_pool2d: too many tiles (%lld)", blocks);
        const size_t lds = (size_t)((R - 1) * stride + size) * row_bytes;
        const int vec = (W % 4 == 0) && aligned16(x);
#define AG_POOL_FWD(SZ, ST)                                                                                   \
    hipLaunchKernelGGL((maxpool_fwd_lds_kernel<SZ, ST>), dim3((unsigned)blocks), dim3(256), lds, as_stream(stream), \
                       x, y, argmax, taps, g, R, bands, vec)
        if (size == 3 && stride == 2) AG_POOL_FWD(3, 2);
        else if (size == 2 && stride == 2) AG_POOL_FWD(2, 2);
        else AG_POOL_FWD(0, 0);
#undef AG_POOL_FWD
    } else {
        const int chunks = (g.OH * g.OW + 255) / 256;
        const long long blocks = (long long)B * C * chunks;
        AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "max_pool2d: too many tiles (%lld)", blocks);
        hipLaunchKernelGGL(maxpool_fwd_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), x, y,
                           argmax, taps, g, chunks);
    }
    return check_launch("max_pool2d");
}

extern "C" ag_status_t ag_relu_maxpool2d_2x2_f32(ag_stream_t stream, const float *a, const float *b, const int *bshape, float *r,
                                                 float *y, float *argmax, uint8_t *taps, int B, int C, int H, int W)
{
    PoolGeom g;
    if ((long long)B * C == 0) return AG_OK;
    if (ag_status_t s = pool_geom("relu_max_pool2d", B, C, H, W, 2, 0, 2, &g)) return s;
    AG_REQUIRE(a && r && y && argmax, AG_ERR_INVALID_DIMS, "relu_max_pool2d: null pointer");
    AG_REQUIRE(H % 2 == 0 && W % 2 == 0, AG_ERR_INVALID_DIMS, "relu_max_pool2d: the 2 x 2 windows must tile the %d x %d plane", H, W);
    AG_REQUIRE((reinterpret_cast<uintptr_t>(a) & 7u) == 0 && (reinterpret_cast<uintptr_t>(r) & 7u) == 0, AG_ERR_INVALID_DIMS,
               "relu_max_pool2d: a and r must be 8-byte aligned");
    BiasStrides bs = {0, 0, 0, 0};
    if (b) {
        AG_REQUIRE(bshape, AG_ERR_INVALID_DIMS, "relu_max_pool2d: the extents of b are missing");
        const int shape[4] = {B, C, H, W};
        long long stride = 1, st[4];
        for (int d = 3; d >= 0; --d) {
            AG_REQUIRE(bshape[d] == shape[d] || bshape[d] == 1, AG_ERR_INCOMPATIBLE_SHAPE,
                       "relu_max_pool2d: extent %d of b on axis %d is neither 1 nor %d", bshape[d], d, shape[d]);
            st[d] = bshape[d] == 1 ? 0 : stride;
            stride *= bshape[d];
        }
        bs = BiasStrides{st[0], st[1], st[2], st[3]};
    }
    const long long outputs = (long long)B * C * g.OH * g.OW, blocks = (outputs + 255) / 256;
    AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "relu_max_pool2d: too many tiles (%lld)", blocks);
    hipLaunchKernelGGL(relu_maxpool_tile2_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), a, b, bs, r, y, argmax,
                       taps, g, C, outputs);
    return check_launch("relu_max_pool2d");
}

// RELU: every stored value is multiplied by greater(relu_x, 0) at its position (a template parameter: as a run-time
// test in the store path it cost the stride-2 kernel a quarter of its speed, 0.110 against 0.087 ms).
template <bool RELU>
static ag_status_t maxpool2d_bwd(ag_stream_t stream, const float *gy, const float *argmax, const uint8_t *taps,
                                 const float *relu_x, float *gx, int B, int C, int H, int W, int size, int pad, int stride)
{
    PoolGeom g;
    if ((long long)B * C == 0) return AG_OK;
    if (ag_status_t s = pool_geom("max_pool2d_grad", B, C, H, W, size, pad, stride, &g)) return s;
    AG_REQUIRE(gy && gx && (argmax || taps), AG_ERR_INVALID_DIMS, "max_pool2d_grad: null pointer");
    AG_REQUIRE(!taps || size <= kMaxTapSize, AG_ERR_INVALID_DIMS,
               "max_pool2d_grad: a tap byte addresses windows of up to %d x %d (got %d)", kMaxTapSize, kMaxTapSize, size);
    AG_REQUIRE(taps || (long long)B * C * H * W <= kExactFloatIndexLimit, AG_ERR_INVALID_DIMS,
               "max_pool2d_grad: an f32 cannot hold offsets into %lld elements exactly (> 2^24); pass the tap bytes",
               (long long)B * C * H * W);
    // (rows of whole quads go to the register kernel below, whose 16-byte stores are worth more on large tensors;
    // up to 2^23 elements its set-up is what counts: [128,32,28,28] 10.0 us there, 5 us here)
    const bool small_tensor = (long long)B * C * H * W <= (1LL << 23);
    if (size == 2 && stride == 2 && pad == 0 && H % 2 == 0 && W % 2 == 0 && (W % 4 != 0 || (small_tensor && g_chunk_rows >= 0)) && (reinterpret_cast<uintptr_t>(gx) & 7) == 0 &&
        (reinterpret_cast<uintptr_t>(relu_x) & 7) == 0 && g.OH > 0 && g.OW > 0) {
        const long long outputs = (long long)B * C * g.OH * g.OW, blocks = (outputs + 255) / 256;
        AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "max_pool2d_grad: too many tiles (%lld)", blocks);
        if (taps)
            hipLaunchKernelGGL((maxpool_bwd_tile2_kernel<true, RELU>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), gy,
                               argmax, taps, relu_x, gx, g, outputs);
        else
            hipLaunchKernelGGL((maxpool_bwd_tile2_kernel<false, RELU>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), gy,
                               argmax, taps, relu_x, gx, g, outputs);
        return check_launch("max_pool2d_grad");
    }
    if (stride == 2 && (size == 2 || size == 3) && W % 4 == 0 && W <= 256 && aligned16(gx) && aligned16(relu_x) && g.OH > 0 && g.OW > 0 &&
        (long long)B * C * g.OH < 0x7fffffffLL && (long long)H * W < 0x7fffffffLL) {
        const int rpc = pool_chunk_rows(g.OH), chunks = (g.OH + rpc - 1) / rpc;
        const long long groups = (long long)B * C * chunks;
        const int lpr = lanes_per_row(W);
        long long blocks = (groups + 4 * (64 / lpr) - 1) / (4 * (64 / lpr));
        if (blocks > 1048576) blocks = 1048576;
#define AG_POOL_BWD_S2(EX, SZ, LP)                                                                            \
    hipLaunchKernelGGL((maxpool_bwd_s2_kernel<EX, SZ, LP, RELU>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), \
                       gy, argmax, taps, relu_x, gx, g, rpc, chunks, (unsigned)groups)
#define AG_POOL_BWD_S2_LPR(EX, SZ)                      \
    switch (lpr) {                                      \
        case 4: AG_POOL_BWD_S2(EX, SZ, 4); break;       \
        case 8: AG_POOL_BWD_S2(EX, SZ, 8); break;       \
        case 16: AG_POOL_BWD_S2(EX, SZ, 16); break;     \
        case 32: AG_POOL_BWD_S2(EX, SZ, 32); break;     \
        default: AG_POOL_BWD_S2(EX, SZ, 64); break;     \
    }
        if (taps) {
            if (size == 3) { AG_POOL_BWD_S2_LPR(true, 3) } else { AG_POOL_BWD_S2_LPR(true, 2) }
        } else {
            if (size == 3) { AG_POOL_BWD_S2_LPR(false, 3) } else { AG_POOL_BWD_S2_LPR(false, 2) }
        }
#undef AG_POOL_BWD_S2_LPR
#undef AG_POOL_BWD_S2
        return check_launch("max_pool2d_grad");
    }
    // LDS-staged path: W % 4 == 0 (128-bit stores) and the windows of a band fit the budget
    const long long orow_bytes = (long long)g.OW * 8;  // gy + index per output
    if (W % 4 == 0 && aligned16(gx) && aligned16(relu_x) && g.OH > 0 && g.OW > 0 &&
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
    hipLaunchKernelGGL((maxpool_bwd_lds_kernel<EX, SZ, ST, RELU>), dim3((unsigned)blocks), dim3(256), lds,               \
                       as_stream(stream), gy, argmax, taps, relu_x, gx, g, IR, bands, max_orows)
        const bool s32 = size == 3 && stride == 2, s22 = size == 2 && stride == 2;
        if (taps) {
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
    if (taps)
        hipLaunchKernelGGL((maxpool_bwd_kernel<true, RELU>), dim3((unsigned)blocks), dim3(256), 0,
                           as_stream(stream), gy, argmax, taps, relu_x, gx, g, chunks);
    else
        hipLaunchKernelGGL((maxpool_bwd_kernel<false, RELU>), dim3((unsigned)blocks), dim3(256), 0,
                           as_stream(stream), gy, argmax, taps, relu_x, gx, g, chunks);
    return check_launch("max_pool2d_grad");
}

extern "C" ag_status_t ag_maxpool2d_bwd_f32(ag_stream_t stream, const float *gy, const float *argmax,
                                            const uint8_t *taps, float *gx, int B, int C, int H,
                                            int W, int size, int pad, int stride)
{
    return maxpool2d_bwd<false>(stream, gy, argmax, taps, nullptr, gx, B, C, H, W, size, pad, stride);
}

// MaxPool2DGrad followed by the gradient of the ReLU in front of the pooling (activation_ops.rs:161-166:
// greater(x, 0) * gy; max_pool2d.rs:245-295), the pair every conv -> relu -> pool block back-propagates through,
// in one pass: gx = greater(relu_x, 0) * max_pool2d_grad(gy), with the bits of the two operators run one after the
// other.  relu_x [B, C, H, W]: the ReLU's input (or its output, which has the same sign pattern).
extern "C" ag_status_t ag_maxpool2d_bwd_relu_f32(ag_stream_t stream, const float *gy, const float *argmax,
                                                 const uint8_t *taps, const float *relu_x, float *gx, int B, int C,
                                                 int H, int W, int size, int pad, int stride)
{
    AG_REQUIRE(relu_x || (long long)B * C * H * W == 0, AG_ERR_INVALID_DIMS, "max_pool2d_grad (relu): null pointer");
    return maxpool2d_bwd<true>(stream, gy, argmax, taps, relu_x, gx, B, C, H, W, size, pad, stride);
}

extern "C" ag_status_t ag_maxpool2d_gradgrad_f32(ag_stream_t stream, const float *ggx,
                                                 const float *argmax, const uint8_t *taps,
                                                 float *ggy, int B, int C, int H, int W, int size,
                                                 int pad, int stride)
{
    PoolGeom g;
    if ((long long)B * C == 0) return AG_OK;
    if (ag_status_t s = pool_geom("max_pool2d_grad_grad", B, C, H, W, size, pad, stride, &g)) return s;
    AG_REQUIRE(ggx && ggy && (argmax || taps), AG_ERR_INVALID_DIMS, "max_pool2d_grad_grad: null pointer");
    AG_REQUIRE(!taps || size <= kMaxTapSize, AG_ERR_INVALID_DIMS,
               "max_pool2d_grad_grad: a tap byte addresses windows of up to %d x %d (got %d)", kMaxTapSize, kMaxTapSize, size);
    AG_REQUIRE(taps || (long long)B * C * H * W <= kExactFloatIndexLimit, AG_ERR_INVALID_DIMS,
               "max_pool2d_grad_grad: an f32 cannot hold offsets into %lld elements exactly (> 2^24); pass the tap bytes",
               (long long)B * C * H * W);
    const long long plane_y = (long long)g.OH * g.OW, total_y = plane_y * B * C;
    if (total_y == 0) return AG_OK;
    long long blocks = (total_y + 255) / 256;
    if (blocks > 262144) blocks = 262144;
    if (taps)
        hipLaunchKernelGGL(maxpool_gradgrad_kernel<true>, dim3((unsigned)blocks), dim3(256), 0,
                           as_stream(stream), ggx, argmax, taps, ggy, g, (long long)H * W, plane_y, total_y);
    else
        hipLaunchKernelGGL(maxpool_gradgrad_kernel<false>, dim3((unsigned)blocks), dim3(256), 0,
                           as_stream(stream), ggx, argmax, taps, ggy, g, (long long)H * W, plane_y, total_y);
    return check_launch("max_pool2d_grad_grad");
}
