// im2col (gather) and col2im (gather-form scatter-add) for NCHW f32 images.
//
// Both are pure data movement bound by HBM: im2col reads |x| and writes kh*kw*|x|-ish bytes,
// col2im the reverse.  im2col stages the input rows a band of output rows needs in LDS once
// (zero padding materialised there), then streams kh*kw output planes out of LDS with fully
// coalesced stores.  col2im assigns one thread per destination pixel and sums the at most
// kh*kw source values in (ky, kx) ascending order -- the order in which the reference's
// sequential scatter reaches that pixel (conv_ops/mod.rs:198-219) -- so no atomics are needed
// and the result is bit-identical for identical input.
#include "ag_internal.h"

namespace ag {

struct ConvGeom {
    int C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, OH, OW;
};

constexpr int kIm2colThreads = 256;
constexpr int kIm2colLdsBytes = 32 * 1024;

// One block = one (image, channel) plane x one band of `R` output rows.
// tile[r][cx] holds x[iy0 + r][cx - pw] (0 outside the image), WL floats per row.
template <bool VEC4, bool STREAM>
__global__ __launch_bounds__(kIm2colThreads) void im2col_lds_kernel(
    const float *__restrict__ x, float *__restrict__ cols, ConvGeom g, int R, int bands, int WL)
{
    extern __shared__ float tile[];
    const int tid = threadIdx.x;
    const int band = blockIdx.x % bands;
    const long long plane = blockIdx.x / bands;  // b*C + c
    const int oy0 = band * R;
    const int rows = min(R, g.OH - oy0);
    const int iy0 = oy0 * g.sh - g.ph;
    const int in_rows = (rows - 1) * g.sh + (g.kh - 1) * g.dh + 1;
    const float *xp = x + plane * (long long)g.H * g.W;

    for (int e = tid; e < in_rows * WL; e += kIm2colThreads) {
        const int r = e / WL;
        const int cx = e - r * WL;
        const int iy = iy0 + r;
        const int ix = cx - g.pw;
        float v = 0.f;
        if ((unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W) v = xp[iy * g.W + ix];
        tile[e] = v;
    }
    __syncthreads();

    const long long P = (long long)g.OH * g.OW;
    const int taps = g.kh * g.kw;
    float *out = cols + plane * taps * P + (long long)oy0 * g.OW;
    const int n_out = rows * g.OW;

    if (VEC4) {
        // OW % 4 == 0: four consecutive outputs share a row and every store is 16-byte aligned.
        for (int e = tid * 4; e < n_out; e += kIm2colThreads * 4) {
            const int r = e / g.OW;
            const int ox = e - r * g.OW;
            const float *src = tile + (r * g.sh) * WL + ox * g.sw;
            float *dst = out + e;
            for (int ky = 0; ky < g.kh; ++ky) {
                for (int kx = 0; kx < g.kw; ++kx) {
                    const float *s = src + ky * g.dh * WL + kx * g.dw;
                    float4 v;
                    v.x = s[0];
                    v.y = s[g.sw];
                    v.z = s[2 * g.sw];
                    v.w = s[3 * g.sw];
                    if (STREAM) st_stream(reinterpret_cast<float4 *>(dst), v);
                    else *reinterpret_cast<float4 *>(dst) = v;
                    dst += P;
                }
            }
        }
    } else {
        for (int e = tid; e < n_out; e += kIm2colThreads) {
            const int r = e / g.OW;
            const int ox = e - r * g.OW;
            const float *src = tile + (r * g.sh) * WL + ox * g.sw;
            float *dst = out + e;
            for (int ky = 0; ky < g.kh; ++ky) {
                for (int kx = 0; kx < g.kw; ++kx) {
                    if (STREAM) st_stream(dst, src[ky * g.dh * WL + kx * g.dw]);
                    else *dst = src[ky * g.dh * WL + kx * g.dw];
                    dst += P;
                }
            }
        }
    }
}

// Fallback without LDS staging for rows too wide to stage: one thread per output element.
__global__ __launch_bounds__(256) void im2col_direct_kernel(const float *__restrict__ x,
                                                            float *__restrict__ cols, ConvGeom g,
                                                            long long total)
{
    const long long P = (long long)g.OH * g.OW;
    for (long long i = blockIdx.x * 256LL + threadIdx.x; i < total; i += gridDim.x * 256LL) {
        const long long row = i / P;  // (b*C + c)*taps + tap
        const int p = (int)(i - row * P);
        const int oy = p / g.OW, ox = p - oy * g.OW;
        const int taps = g.kh * g.kw;
        const long long plane = row / taps;
        const int tap = (int)(row - plane * taps);
        const int ky = tap / g.kw, kx = tap - ky * g.kw;
        const int iy = oy * g.sh - g.ph + ky * g.dh;
        const int ix = ox * g.sw - g.pw + kx * g.dw;
        float v = 0.f;
        if ((unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W)
            v = x[plane * (long long)g.H * g.W + iy * g.W + ix];
        cols[i] = v;
    }
}

// One thread per destination pixel (any stride / dilation).
__global__ __launch_bounds__(256) void col2im_gather_kernel(const float *__restrict__ cols,
                                                            float *__restrict__ gx, ConvGeom g,
                                                            int chunks)
{
    const int chunk = blockIdx.x % chunks;
    const long long plane = blockIdx.x / chunks;
    const int HW = g.H * g.W;
    const int e = chunk * 256 + threadIdx.x;
    if (e >= HW) return;
    const int iy = e / g.W, ix = e - iy * g.W;
    const long long P = (long long)g.OH * g.OW;
    const float *cp = cols + plane * (long long)(g.kh * g.kw) * P;
    float acc = 0.f;
    for (int ky = 0; ky < g.kh; ++ky) {
        const int ty = iy + g.ph - ky * g.dh;
        if (ty < 0) break;  // later ky only lowers ty
        const int oy = ty / g.sh;
        if (oy * g.sh != ty || oy >= g.OH) continue;
        for (int kx = 0; kx < g.kw; ++kx) {
            const int tx = ix + g.pw - kx * g.dw;
            if (tx < 0) break;
            const int ox = tx / g.sw;
            if (ox * g.sw != tx || ox >= g.OW) continue;
            acc += cp[(long long)(ky * g.kw + kx) * P + oy * g.OW + ox];
        }
    }
    gx[plane * HW + e] = acc;
}

// The same for a 3 x 3 filter at stride 1 and any dilation: the nine tap addresses are computed and their
// loads issued together (absent taps read nothing and add 0.0, which leaves the sum unchanged), then
// added in (ky, kx) ascending order.  The run-time loops of the general kernel issue one load at a time.
__global__ __launch_bounds__(256) void col2im_gather3_kernel(const float *__restrict__ cols, float *__restrict__ gx,
                                                             ConvGeom g, int chunks)
{
    const int chunk = blockIdx.x % chunks;
    const long long plane = blockIdx.x / chunks;
    const int HW = g.H * g.W;
    const int e = chunk * 256 + threadIdx.x;
    if (e >= HW) return;
    const int iy = e / g.W, ix = e - iy * g.W;
    const long long P = (long long)g.OH * g.OW;
    const float *cp = cols + plane * 9 * P;
    float v[9];
#pragma unroll
    for (int ky = 0; ky < 3; ++ky) {
        const int oy = iy + g.ph - ky * g.dh;
#pragma unroll
        for (int kx = 0; kx < 3; ++kx) {
            const int ox = ix + g.pw - kx * g.dw;
            const bool in = (unsigned)oy < (unsigned)g.OH && (unsigned)ox < (unsigned)g.OW;
            v[ky * 3 + kx] = in ? cp[(long long)(ky * 3 + kx) * P + oy * g.OW + ox] : 0.f;
        }
    }
    float acc = 0.f;
#pragma unroll
    for (int t = 0; t < 9; ++t) acc += v[t];
    gx[plane * HW + e] = acc;
}

// 16 bytes that are only 4-byte aligned (the hardware handles the misalignment).
struct __attribute__((packed, aligned(4))) Float4U {
    float x, y, z, w;
};

// Stride 1, W % 4 == 0: one thread per four consecutive destination pixels of a row.  Each of
// the kh*kw taps is one (generally misaligned) 128-bit load from its plane of the columns; the
// four sums keep the (ky, kx) ascending order of the reference.  Groups that touch the left or
// right border take per-pixel loads.
template <int KH, int KW>  // 0 = run-time extents
__global__ __launch_bounds__(256) void col2im_unit_vec4_kernel(const float *__restrict__ cols,
                                                               float *__restrict__ gx, ConvGeom g,
                                                               long long groups)
{
    const int kh = KH ? KH : g.kh, kw = KW ? KW : g.kw;
    const int W4 = g.W >> 2;
    const long long P = (long long)g.OH * g.OW;
    const long long taps_stride = (long long)(kh * kw) * P;
    for (long long gi = blockIdx.x * 256LL + threadIdx.x; gi < groups; gi += gridDim.x * 256LL) {
        const long long row = gi / W4;  // (plane, iy)
        const int ix0 = (int)(gi - row * W4) * 4;
        const long long plane = row / g.H;
        const int iy = (int)(row - plane * g.H);
        const float *cp = cols + plane * taps_stride;
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
        for (int ky = 0; ky < kh; ++ky) {
            const int oy = iy + g.ph - ky * g.dh;
            if ((unsigned)oy >= (unsigned)g.OH) continue;
#pragma unroll
            for (int kx = 0; kx < kw; ++kx) {
                const int ox0 = ix0 + g.pw - kx * g.dw;
                const float *src = cp + (long long)(ky * kw + kx) * P + (long long)oy * g.OW + ox0;
                if (ox0 >= 0 && ox0 + 3 < g.OW) {
                    const Float4U v = *reinterpret_cast<const Float4U *>(src);  // read once, misaligned
                    a0 += v.x;
                    a1 += v.y;
                    a2 += v.z;
                    a3 += v.w;
                } else {
                    if ((unsigned)(ox0 + 0) < (unsigned)g.OW) a0 += src[0];
                    if ((unsigned)(ox0 + 1) < (unsigned)g.OW) a1 += src[1];
                    if ((unsigned)(ox0 + 2) < (unsigned)g.OW) a2 += src[2];
                    if ((unsigned)(ox0 + 3) < (unsigned)g.OW) a3 += src[3];
                }
            }
        }
        st_stream(reinterpret_cast<float4 *>(gx + gi * 4), make_float4(a0, a1, a2, a3));
    }
}

// Stride 1, dilation 1 along x, output as wide as the input (W == OW, W % 4 == 0, W <= 256): the
// "same"-size convolutions.  LPR lanes (a power of two >= W/4) share one destination row, each
// owning four consecutive pixels.  Every tap plane is read with ALIGNED 128-bit streaming loads
// at the lane's own four columns; the horizontal shift of the tap (pw - kx, between -3 and 3) is
// applied afterwards by taking the missing column(s) from the neighbouring lane, zero outside
// the row.  All kh*kw loads of a thread are issued before the first use.  The sums keep the
// (ky, kx) ascending order of the reference.
template <int KH, int KW, int PW, int LPR>
__global__ __launch_bounds__(256) void col2im_same_kernel(const float *__restrict__ cols, float *__restrict__ gx,
                                                          ConvGeom g, unsigned rows_total)
{
    constexpr int RPW = 64 / LPR;  // rows per wave
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int q = lane & (LPR - 1);
    const int W4 = g.W >> 2;
    const bool in_row = q < W4;
    const unsigned P = (unsigned)(g.OH * g.OW);
    for (unsigned r = (blockIdx.x * 4u + wave) * RPW + lane / LPR; r - lane / LPR < rows_total;
         r += gridDim.x * 4u * RPW) {
        const bool active = in_row && r < rows_total;
        const unsigned plane = r / (unsigned)g.H;
        const int iy = (int)(r - plane * (unsigned)g.H);
        const float *cp = cols + (long long)plane * (KH * KW) * P + q * 4;
        float4 v[KH][KW];
#pragma unroll
        for (int ky = 0; ky < KH; ++ky) {
            const int oy = iy + g.ph - ky * g.dh;
            const bool ok = active && (unsigned)oy < (unsigned)g.OH;
#pragma unroll
            for (int kx = 0; kx < KW; ++kx)
                v[ky][kx] = ok ? ld_stream(reinterpret_cast<const float4 *>(cp + (unsigned)(ky * KW + kx) * P + (unsigned)oy * g.OW))
                               : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
        for (int ky = 0; ky < KH; ++ky)
#pragma unroll
            for (int kx = 0; kx < KW; ++kx) {
                const int d = PW - kx;  // source column = destination column + d
                const float4 c = v[ky][kx];
                if (d == 0) {
                    a0 += c.x; a1 += c.y; a2 += c.z; a3 += c.w;
                } else if (d > 0) {
                    // columns 4q+d .. 4q+d+3: own elements d..3, then the next lane's 0..d-1
                    const bool has = q + 1 < W4;
                    const float nx = __shfl_down(c.x, 1, LPR), ny = __shfl_down(c.y, 1, LPR), nz = __shfl_down(c.z, 1, LPR);
                    const float e0 = has ? nx : 0.f, e1 = has ? ny : 0.f, e2 = has ? nz : 0.f;
                    if (d == 1) { a0 += c.y; a1 += c.z; a2 += c.w; a3 += e0; }
                    else if (d == 2) { a0 += c.z; a1 += c.w; a2 += e0; a3 += e1; }
                    else { a0 += c.w; a1 += e0; a2 += e1; a3 += e2; }
                } else {
                    // columns 4q+d .. : the previous lane's last -d elements, then own 0..3+d
                    const bool has = q > 0;
                    const float py = __shfl_up(c.y, 1, LPR), pz = __shfl_up(c.z, 1, LPR), pw_ = __shfl_up(c.w, 1, LPR);
                    const float e1 = has ? py : 0.f, e2 = has ? pz : 0.f, e3 = has ? pw_ : 0.f;
                    if (d == -1) { a0 += e3; a1 += c.x; a2 += c.y; a3 += c.z; }
                    else if (d == -2) { a0 += e2; a1 += e3; a2 += c.x; a3 += c.y; }
                    else { a0 += e1; a1 += e2; a2 += e3; a3 += c.x; }
                }
            }
        if (active) st_stream(reinterpret_cast<float4 *>(gx + (long long)r * g.W + q * 4), make_float4(a0, a1, a2, a3));
    }
}

template <int KH, int KW, int PW>
static void launch_col2im_same(hipStream_t st, const float *cols, float *gx, const ConvGeom &g, long long rows)
{
    const int W4 = g.W >> 2;
    const int lpr = W4 <= 4 ? 4 : W4 <= 8 ? 8 : W4 <= 16 ? 16 : W4 <= 32 ? 32 : 64;
    const long long rows_per_block = 4 * (64 / lpr);
    long long blocks = (rows + rows_per_block - 1) / rows_per_block;
    if (blocks > 1048576) blocks = 1048576;
    const dim3 grid((unsigned)blocks), block(256);
    switch (lpr) {
        case 4: hipLaunchKernelGGL((col2im_same_kernel<KH, KW, PW, 4>), grid, block, 0, st, cols, gx, g, (unsigned)rows); break;
        case 8: hipLaunchKernelGGL((col2im_same_kernel<KH, KW, PW, 8>), grid, block, 0, st, cols, gx, g, (unsigned)rows); break;
        case 16: hipLaunchKernelGGL((col2im_same_kernel<KH, KW, PW, 16>), grid, block, 0, st, cols, gx, g, (unsigned)rows); break;
        case 32: hipLaunchKernelGGL((col2im_same_kernel<KH, KW, PW, 32>), grid, block, 0, st, cols, gx, g, (unsigned)rows); break;
        default: hipLaunchKernelGGL((col2im_same_kernel<KH, KW, PW, 64>), grid, block, 0, st, cols, gx, g, (unsigned)rows); break;
    }
}

// Stride 2 on both axes: one thread per 2x2 block of destination pixels.  Every tap (ky, kx)
// feeds exactly one pixel of the block (the one whose offset has the right parity), so a thread
// reads each of the kh*kw planes once, at consecutive positions for consecutive threads, and no
// lane idles on a divisibility test.  Taps are visited in (ky, kx) ascending order, so each
// pixel still receives its terms in the reference's order.
__global__ __launch_bounds__(256) void col2im_stride2_kernel(const float *__restrict__ cols,
                                                             float *__restrict__ gx, ConvGeom g,
                                                             long long nblk)
{
    const int BW = (g.W + 1) >> 1, BH = (g.H + 1) >> 1;
    const long long P = (long long)g.OH * g.OW;
    for (long long gi = blockIdx.x * 256LL + threadIdx.x; gi < nblk; gi += gridDim.x * 256LL) {
        const long long rowi = gi / BW;  // (plane, by)
        const int bx = (int)(gi - rowi * BW);
        const long long plane = rowi / BH;
        const int by = (int)(rowi - plane * BH);
        const float *cp = cols + plane * (long long)(g.kh * g.kw) * P;
        float a00 = 0.f, a01 = 0.f, a10 = 0.f, a11 = 0.f;
        for (int ky = 0; ky < g.kh; ++ky) {
            const int ry = (ky * g.dh - g.ph) & 1;  // parity of the row this tap feeds
            const int ty = 2 * by + ry + g.ph - ky * g.dh;
            const int oy = ty >> 1;
            const bool vy = ty >= 0 && oy < g.OH;
            for (int kx = 0; kx < g.kw; ++kx) {
                const int rx = (kx * g.dw - g.pw) & 1;
                const int tx = 2 * bx + rx + g.pw - kx * g.dw;
                const int ox = tx >> 1;
                if (vy && tx >= 0 && ox < g.OW) {
                    const float v = cp[(long long)(ky * g.kw + kx) * P + (long long)oy * g.OW + ox];
                    if (ry == 0) {
                        if (rx == 0) a00 += v;
                        else a01 += v;
                    } else {
                        if (rx == 0) a10 += v;
                        else a11 += v;
                    }
                }
            }
        }
        float *dst = gx + plane * (long long)g.H * g.W + (long long)(2 * by) * g.W + 2 * bx;
        const bool c1 = 2 * bx + 1 < g.W, r1 = 2 * by + 1 < g.H;
        dst[0] = a00;
        if (c1) dst[1] = a01;
        if (r1) {
            dst[g.W] = a10;
            if (c1) dst[g.W + 1] = a11;
        }
    }
}

// The same for the usual geometries (dilation 1, W and H even) with the window and the padding known
// at compile time: no run-time loops or parity tests, 32-bit offsets inside a plane, one streaming
// load per tap (consecutive lanes read consecutive positions) and two 64-bit streaming stores (the
// lanes of a wave write 512 contiguous bytes per row).  Same visiting order.
template <int KH, int KW, int PH, int PW>
__global__ __launch_bounds__(256) void col2im_stride2_vec_kernel(const float *__restrict__ cols,
                                                                 float *__restrict__ gx, ConvGeom g,
                                                                 unsigned nblk)
{
    const unsigned gi = blockIdx.x * 256u + threadIdx.x;
    if (gi >= nblk) return;
    const unsigned BW = (unsigned)g.W >> 1, BH = (unsigned)g.H >> 1;
    const unsigned rowi = gi / BW, bx = gi - rowi * BW;  // (plane, by)
    const unsigned plane = rowi / BH, by = rowi - plane * BH;
    const unsigned P = (unsigned)(g.OH * g.OW);
    const float *cp = cols + (long long)plane * (KH * KW) * P;
    float acc[2][2] = {};
#pragma unroll
    for (int ky = 0; ky < KH; ++ky) {
        const int ry = (ky - PH) & 1;
        const int ty = 2 * (int)by + ry + PH - ky;
        const int oy = ty >> 1;
        const bool vy = ty >= 0 && oy < g.OH;
#pragma unroll
        for (int kx = 0; kx < KW; ++kx) {
            const int rx = (kx - PW) & 1;
            const int tx = 2 * (int)bx + rx + PW - kx;
            const int ox = tx >> 1;
            if (vy && tx >= 0 && ox < g.OW) acc[ry][rx] += ld_stream(cp + (unsigned)(ky * KW + kx) * P + oy * g.OW + ox);
        }
    }
    float *dst = gx + (long long)plane * g.H * g.W + (2 * by) * (unsigned)g.W + 2 * bx;
    *reinterpret_cast<float2 *>(dst) = make_float2(acc[0][0], acc[0][1]);
    *reinterpret_cast<float2 *>(dst + g.W) = make_float2(acc[1][0], acc[1][1]);
}

// Stride 2, 3x3 window, pad 1, dilation 1 on an even image (W == 2 * OW, OW % 4 == 0): a thread
// owns four consecutive outputs of one row.  Per window row it loads the nine input elements they
// touch (two aligned 128-bit loads and the element to their left), picks the three column phases
// out of registers and streams one aligned 128-bit store per tap.  No LDS, no run-time loops.
__global__ __launch_bounds__(256) void im2col_s2_k3_kernel(const float *__restrict__ x, float *__restrict__ cols,
                                                           ConvGeom g, unsigned ngroups)
{
    const unsigned gi = blockIdx.x * 256u + threadIdx.x;
    if (gi >= ngroups) return;
    const unsigned OW4 = (unsigned)g.OW >> 2;
    const unsigned rowi = gi / OW4, q = gi - rowi * OW4;  // (plane, oy), group of four outputs
    const unsigned plane = rowi / (unsigned)g.OH, oy = rowi - plane * (unsigned)g.OH;
    const unsigned P = (unsigned)(g.OH * g.OW);
    const float *xp = x + (long long)plane * g.H * g.W;
    float *dst = cols + (long long)plane * 9 * P + oy * (unsigned)g.OW + 4 * q;
    const int ix0 = 8 * (int)q;  // first even column; the window of output ox starts at 2*ox - 1
#pragma unroll
    for (int ky = 0; ky < 3; ++ky) {
        const int iy = 2 * (int)oy + ky - 1;
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
        float left = 0.f;
        if ((unsigned)iy < (unsigned)g.H) {
            const float *row = xp + iy * g.W + ix0;
            a = *reinterpret_cast<const float4 *>(row);
            b = *reinterpret_cast<const float4 *>(row + 4);
            if (ix0 > 0) left = row[-1];
        }
        st_stream(reinterpret_cast<float4 *>(dst + (unsigned)(ky * 3 + 0) * P), make_float4(left, a.y, a.w, b.y));
        st_stream(reinterpret_cast<float4 *>(dst + (unsigned)(ky * 3 + 1) * P), make_float4(a.x, a.z, b.x, b.z));
        st_stream(reinterpret_cast<float4 *>(dst + (unsigned)(ky * 3 + 2) * P), make_float4(a.y, a.w, b.y, b.w));
    }
}

static ag_status_t check_geom(const char *who, int B, int C, int H, int W, int kh, int kw, int ph,
                              int pw, int sh, int sw, int dh, int dw)
{
    AG_REQUIRE(B >= 0 && C >= 0 && H >= 0 && W >= 0, AG_ERR_INVALID_DIMS,
               "%s: negative extent (B=%d C=%d H=%d W=%d)", who, B, C, H, W);
    AG_REQUIRE(kh >= 1 && kw >= 1 && sh >= 1 && sw >= 1 && dh >= 1 && dw >= 1 && ph >= 0 && pw >= 0,
               AG_ERR_INVALID_DIMS,
               "%s: kernel/stride/dilation must be >= 1 and pad >= 0 (k=%dx%d s=%dx%d d=%dx%d p=%dx%d)",
               who, kh, kw, sh, sw, dh, dw, ph, pw);
    return AG_OK;
}

// im2col for the "same"-size stride-1 convolutions (W == OW, W % 4 == 0, W <= 256, dilation 1
// along x): the mirror image of col2im_same_kernel.  LPR lanes share one output row, each owning
// four consecutive columns.  A lane loads its own four columns of the kh input rows with aligned
// 128-bit loads (zero outside the image), builds the kw horizontally shifted versions with one
// lane exchange each, and streams the kh*kw results to their planes with aligned 128-bit
// non-temporal stores.  No LDS, no divisions besides one per thread.
template <int KH, int KW, int PW, int LPR>
__global__ __launch_bounds__(256) void im2col_same_kernel(const float *__restrict__ x, float *__restrict__ cols,
                                                          ConvGeom g, unsigned rows_total)
{
    constexpr int RPW = 64 / LPR;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int q = lane & (LPR - 1);
    const int W4 = g.W >> 2;
    const bool in_row = q < W4;
    const unsigned P = (unsigned)(g.OH * g.OW);
    for (unsigned r = (blockIdx.x * 4u + wave) * RPW + lane / LPR; r - lane / LPR < rows_total;
         r += gridDim.x * 4u * RPW) {
        const bool active = in_row && r < rows_total;
        const unsigned plane = r / (unsigned)g.OH;
        const int oy = (int)(r - plane * (unsigned)g.OH);
        const float *xp = x + (long long)plane * g.H * g.W + q * 4;
        float4 v[KH];
#pragma unroll
        for (int ky = 0; ky < KH; ++ky) {
            const int iy = oy - g.ph + ky * g.dh;
            const bool ok = active && (unsigned)iy < (unsigned)g.H;
            v[ky] = ok ? *reinterpret_cast<const float4 *>(xp + (unsigned)iy * g.W) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        float *cp = cols + (long long)plane * (KH * KW) * P + (unsigned)oy * g.OW + q * 4;
#pragma unroll
        for (int ky = 0; ky < KH; ++ky)
#pragma unroll
            for (int kx = 0; kx < KW; ++kx) {
                const int d = kx - PW;  // source column = output column + d
                const float4 c = v[ky];
                float4 o;
                if (d == 0) {
                    o = c;
                } else if (d > 0) {
                    const bool has = q + 1 < W4;
                    const float nx = __shfl_down(c.x, 1, LPR), ny = __shfl_down(c.y, 1, LPR), nz = __shfl_down(c.z, 1, LPR);
                    const float e0 = has ? nx : 0.f, e1 = has ? ny : 0.f, e2 = has ? nz : 0.f;
                    if (d == 1) o = make_float4(c.y, c.z, c.w, e0);
                    else if (d == 2) o = make_float4(c.z, c.w, e0, e1);
                    else o = make_float4(c.w, e0, e1, e2);
                } else {
                    const bool has = q > 0;
                    const float py = __shfl_up(c.y, 1, LPR), pz = __shfl_up(c.z, 1, LPR), pw_ = __shfl_up(c.w, 1, LPR);
                    const float e1 = has ? py : 0.f, e2 = has ? pz : 0.f, e3 = has ? pw_ : 0.f;
                    if (d == -1) o = make_float4(e3, c.x, c.y, c.z);
                    else if (d == -2) o = make_float4(e2, e3, c.x, c.y);
                    else o = make_float4(e1, e2, e3, c.x);
                }
                if (active) st_stream(reinterpret_cast<float4 *>(cp + (unsigned)(ky * KW + kx) * P), o);
            }
    }
}

template <int KH, int KW, int PW>
static void launch_im2col_same(hipStream_t st, const float *x, float *cols, const ConvGeom &g, long long rows)
{
    const int W4 = g.W >> 2;
    const int lpr = W4 <= 4 ? 4 : W4 <= 8 ? 8 : W4 <= 16 ? 16 : W4 <= 32 ? 32 : 64;
    const long long rows_per_block = 4 * (64 / lpr);
    long long blocks = (rows + rows_per_block - 1) / rows_per_block;
    if (blocks > 1048576) blocks = 1048576;
    const dim3 grid((unsigned)blocks), block(256);
    switch (lpr) {
        case 4: hipLaunchKernelGGL((im2col_same_kernel<KH, KW, PW, 4>), grid, block, 0, st, x, cols, g, (unsigned)rows); break;
        case 8: hipLaunchKernelGGL((im2col_same_kernel<KH, KW, PW, 8>), grid, block, 0, st, x, cols, g, (unsigned)rows); break;
        case 16: hipLaunchKernelGGL((im2col_same_kernel<KH, KW, PW, 16>), grid, block, 0, st, x, cols, g, (unsigned)rows); break;
        case 32: hipLaunchKernelGGL((im2col_same_kernel<KH, KW, PW, 32>), grid, block, 0, st, x, cols, g, (unsigned)rows); break;
        default: hipLaunchKernelGGL((im2col_same_kernel<KH, KW, PW, 64>), grid, block, 0, st, x, cols, g, (unsigned)rows); break;
    }
}

}  // namespace ag

using namespace ag;

extern "C" ag_status_t ag_im2col_f32(ag_stream_t stream, const float *x, float *cols, int B, int C,
                                     int H, int W, int kh, int kw, int ph, int pw, int sh, int sw,
                                     int dh, int dw)
{
    if (ag_status_t s = check_geom("im2col", B, C, H, W, kh, kw, ph, pw, sh, sw, dh, dw)) return s;
    const int OH = ag_conv_out_size(H, kh, ph, sh, dh);
    const int OW = ag_conv_out_size(W, kw, pw, sw, dw);
    AG_REQUIRE(H + 2 * ph >= dh * (kh - 1) + 1 && W + 2 * pw >= dw * (kw - 1) + 1,
               AG_ERR_INVALID_DIMS, "im2col: kernel extent exceeds the padded image (%dx%d, k=%dx%d d=%dx%d p=%dx%d)",
               H, W, kh, kw, dh, dw, ph, pw);
    const long long planes = (long long)B * C;
    if (planes == 0 || OH <= 0 || OW <= 0) return AG_OK;
    AG_REQUIRE(x && cols, AG_ERR_INVALID_DIMS, "im2col: null pointer");
    ConvGeom g{C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, OH, OW};

    const bool same = sh == 1 && sw == 1 && dw == 1 && OW == W && ph == pw && W % 4 == 0 && W <= 256 &&
                      aligned16(x) && aligned16(cols) && planes * OH < 0x7fffffffLL &&
                      (long long)kh * kw * OH * OW < 0x7fffffffLL && (long long)H * W < 0x7fffffffLL;
    if (same && kh == 3 && kw == 3 && pw == 1) {
        launch_im2col_same<3, 3, 1>(as_stream(stream), x, cols, g, planes * OH);
        return check_launch("im2col");
    }
    if (same && kh == 5 && kw == 5 && pw == 2) {
        launch_im2col_same<5, 5, 2>(as_stream(stream), x, cols, g, planes * OH);
        return check_launch("im2col");
    }

    if (sh == 2 && sw == 2 && dh == 1 && dw == 1 && kh == 3 && kw == 3 && ph == 1 && pw == 1 && W == 2 * OW && OW % 4 == 0 &&
        aligned16(x) && aligned16(cols) && planes * OH * (OW / 4) < 0xffffffffLL && 9LL * OH * OW < 0x7fffffffLL &&
        (long long)H * W < 0x7fffffffLL) {
        const unsigned ngroups = (unsigned)(planes * OH * (OW / 4));
        hipLaunchKernelGGL(im2col_s2_k3_kernel, dim3((ngroups + 255) / 256), dim3(256), 0, as_stream(stream), x, cols, g, ngroups);
        return check_launch("im2col");
    }

    const int WL = (OW - 1) * sw + (kw - 1) * dw + 1;  // staged row length
    const int rows_min = (kh - 1) * dh + 1;            // input rows for one output row
    const long long lds_one = (long long)rows_min * WL * 4;
    if (lds_one <= kIm2colLdsBytes) {
        // Band height: many small blocks keep more independent store streams in flight than a
        // few long-running ones, but every band re-stages (kh-1)*dh halo rows, which costs more
        // the larger the stride.  Aim at 448*sh*sw outputs per tap and block (8 rows of 56 at
        // stride 1 measured best inside the conv step), capped by the LDS budget.
        int R = (int)((kIm2colLdsBytes / 4 / WL - rows_min) / sh + 1);
        const int want = (448 * sh * sw + OW - 1) / OW;
        if (R > want) R = want;
        if (R > OH) R = OH;
        if (R < 1) R = 1;
        const int bands = (OH + R - 1) / R;
        const long long blocks = planes * bands;
        AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "im2col: too many tiles (%lld)", blocks);
        const size_t lds = (size_t)((R - 1) * sh + rows_min) * WL * 4;
        const bool vec4 = (OW % 4 == 0) && aligned16(cols);
        const bool strm = true;  // streaming stores: cols is far larger than the caches
#define AG_IM2COL_LAUNCH(V, S)                                                                           \
    hipLaunchKernelGGL((im2col_lds_kernel<V, S>), dim3((unsigned)blocks), dim3(kIm2colThreads), lds,      \
                       as_stream(stream), x, cols, g, R, bands, WL)
        if (vec4 && strm) AG_IM2COL_LAUNCH(true, true);
        else if (vec4) AG_IM2COL_LAUNCH(true, false);
        else if (strm) AG_IM2COL_LAUNCH(false, true);
        else AG_IM2COL_LAUNCH(false, false);
#undef AG_IM2COL_LAUNCH
    } else {
        const long long total = planes * kh * kw * (long long)OH * OW;
        long long blocks = (total + 255) / 256;
        if (blocks > 1048576) blocks = 1048576;
        hipLaunchKernelGGL(im2col_direct_kernel, dim3((unsigned)blocks), dim3(256), 0,
                           as_stream(stream), x, cols, g, total);
    }
    return check_launch("im2col");
}

extern "C" ag_status_t ag_col2im_f32(ag_stream_t stream, const float *cols, float *gx, int B, int C,
                                     int H, int W, int kh, int kw, int ph, int pw, int sh, int sw,
                                     int dh, int dw, int OH, int OW)
{
    if (ag_status_t s = check_geom("col2im", B, C, H, W, kh, kw, ph, pw, sh, sw, dh, dw)) return s;
    AG_REQUIRE(OH >= 0 && OW >= 0, AG_ERR_INVALID_DIMS, "col2im: negative output extent (%dx%d)", OH, OW);
    const long long planes = (long long)B * C;
    if (planes == 0 || H == 0 || W == 0) return AG_OK;
    AG_REQUIRE(gx && (cols || OH == 0 || OW == 0), AG_ERR_INVALID_DIMS, "col2im: null pointer");
    AG_REQUIRE((long long)H * W <= 0x7fffffffLL, AG_ERR_INVALID_DIMS, "col2im: plane too large");
    ConvGeom g{C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, OH, OW};
    const bool same = sh == 1 && sw == 1 && dw == 1 && OW == W && W % 4 == 0 && W <= 256 && aligned16(gx) &&
                      aligned16(cols) && planes * H < 0x7fffffffLL && (long long)kh * kw * OH * OW < 0x7fffffffLL;
    if (same && kh == 3 && kw == 3 && pw == 1) {
        launch_col2im_same<3, 3, 1>(as_stream(stream), cols, gx, g, planes * H);
    } else if (same && kh == 5 && kw == 5 && pw == 2) {
        launch_col2im_same<5, 5, 2>(as_stream(stream), cols, gx, g, planes * H);
    } else if (sh == 1 && sw == 1 && W % 4 == 0 && aligned16(gx)) {
        const long long groups = planes * H * (W / 4);
        long long blocks = (groups + 255) / 256;
        if (blocks > 262144) blocks = 262144;
        if (kh == 3 && kw == 3)
            hipLaunchKernelGGL((col2im_unit_vec4_kernel<3, 3>), dim3((unsigned)blocks), dim3(256), 0,
                               as_stream(stream), cols, gx, g, groups);
        else
            hipLaunchKernelGGL((col2im_unit_vec4_kernel<0, 0>), dim3((unsigned)blocks), dim3(256), 0,
                               as_stream(stream), cols, gx, g, groups);
    } else if (sh == 2 && sw == 2 && dh == 1 && dw == 1 && W % 2 == 0 && H % 2 == 0 && (reinterpret_cast<uintptr_t>(gx) & 7u) == 0 &&
               ((kh == 3 && kw == 3) || (kh == 4 && kw == 4)) && ph == 1 && pw == 1 &&
               planes * (H / 2) * (W / 2) < 0xffffffffLL && (long long)kh * kw * OH * OW < 0x7fffffffLL) {
        const unsigned nblk = (unsigned)(planes * (H / 2) * (W / 2));
        const dim3 grid((nblk + 255) / 256), block(256);
        if (kh == 3)
            hipLaunchKernelGGL((col2im_stride2_vec_kernel<3, 3, 1, 1>), grid, block, 0, as_stream(stream), cols, gx, g, nblk);
        else
            hipLaunchKernelGGL((col2im_stride2_vec_kernel<4, 4, 1, 1>), grid, block, 0, as_stream(stream), cols, gx, g, nblk);
    } else if (sh == 2 && sw == 2) {
        const long long nblk = planes * ((H + 1) / 2) * ((W + 1) / 2);
        long long blocks = (nblk + 255) / 256;
        if (blocks > 1048576) blocks = 1048576;
        hipLaunchKernelGGL(col2im_stride2_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), cols,
                           gx, g, nblk);
    } else {
        const int chunks = (H * W + 255) / 256;
        const long long blocks = planes * chunks;
        AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "col2im: too many tiles (%lld)", blocks);
        if (kh == 3 && kw == 3 && sh == 1 && sw == 1)
            hipLaunchKernelGGL(col2im_gather3_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), cols, gx, g,
                               chunks);
        else
            hipLaunchKernelGGL(col2im_gather_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), cols,
                               gx, g, chunks);
    }
    return check_launch("col2im");
}
