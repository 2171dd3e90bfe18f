// Convolution operators as compositions of im2col / col2im and the MFMA GEMM, mirroring how the
// reference builds them (conv2d.rs:25-112, 631-734; conv2d_transpose.rs:89-247, 303-431) but
// batched: one im2col launch and one strided-batched GEMM launch per operator instead of one
// task per image, and one split-accumulation GEMM instead of an image-sequential beta=1 loop.
#include "ag_internal.h"
#include "conv_shared.h"
#include "gemm_shared.h"

using namespace ag;

static ag_status_t conv_dims(const char *who, int B, int C, int H, int W, int K, int kh, int kw, int pad,
                             int stride, int dilation)
{
    AG_REQUIRE(B >= 0 && C >= 0 && H >= 0 && W >= 0 && K >= 0, AG_ERR_INVALID_DIMS,
               "%s: negative extent (B=%d C=%d H=%d W=%d K=%d)", who, B, C, H, W, K);
    AG_REQUIRE(kh >= 1 && kw >= 1 && stride >= 1 && dilation >= 1 && pad >= 0, AG_ERR_INVALID_DIMS,
               "%s: kernel/stride/dilation must be >= 1 and pad >= 0 (k=%dx%d stride=%d dilation=%d pad=%d)", who,
               kh, kw, stride, dilation, pad);
    return AG_OK;
}

namespace ag {

// Forward product of a thin first layer, y_b[K x P] = w[K x CK] . cols_b[CK x P] with CK <= 16 (e.g. the
// 1 -> 32 channel 3x3 convolution of the small CNN: CK = 9).  A tiled GEMM spends its time on a k-tile that is
// mostly padding; here the kernel is the HBM-bound copy it should be: a thread holds the CK column values of four
// neighbouring positions in registers and writes one 128-bit result per filter for a pair of filters
// (the filter taps, padded to 16 per filter with zeros, sit in LDS).  Products are added in tap order.
constexpr int kThinFwdMaxCK = 16, kThinFwdGroup = 2;

__global__ __launch_bounds__(256) void thin_fwd_kernel(const float *__restrict__ cols, const float *__restrict__ w,
                                                       float *__restrict__ y, int CK, int P4, int K, long long quads)
{
    __shared__ float s_w[kThinFwdGroup * kThinFwdMaxCK];
    const int k0 = blockIdx.y * kThinFwdGroup;
    const long long q = blockIdx.x * 256ll + threadIdx.x;
    const bool active = q < quads;
    const long long b = active ? q / P4 : 0;
    const int p4 = active ? (int)(q - b * P4) : 0;
    // the column loads go out before the filter taps are staged: both round trips overlap
    const float4 *cb = reinterpret_cast<const float4 *>(cols) + b * CK * (long long)P4 + p4;
    float4 c[kThinFwdMaxCK];
#pragma unroll
    for (int j = 0; j < kThinFwdMaxCK; ++j) c[j] = (active && j < CK) ? cb[(long long)j * P4] : make_float4(0.f, 0.f, 0.f, 0.f);
    if (threadIdx.x < kThinFwdGroup * kThinFwdMaxCK) {
        const int k = k0 + threadIdx.x / kThinFwdMaxCK, j = threadIdx.x % kThinFwdMaxCK;
        s_w[threadIdx.x] = (k < K && j < CK) ? w[k * CK + j] : 0.f;
    }
    __syncthreads();
    if (!active) return;
    float4 *yb = reinterpret_cast<float4 *>(y) + (b * K + k0) * (long long)P4 + p4;
#pragma unroll
    for (int g = 0; g < kThinFwdGroup; ++g) {
        if (k0 + g >= K) break;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int j = 0; j < kThinFwdMaxCK; ++j) {
            const float wv = s_w[g * kThinFwdMaxCK + j];
            acc.x = fmaf(wv, c[j].x, acc.x);
            acc.y = fmaf(wv, c[j].y, acc.y);
            acc.z = fmaf(wv, c[j].z, acc.z);
            acc.w = fmaf(wv, c[j].w, acc.w);
        }
        yb[(long long)g * P4] = acc;
    }
}

// Takes the product when it fits the kernel; false = the caller runs the GEMM.
static bool thin_fwd(hipStream_t st, const float *cols, const float *w, float *y, int B, long long CK, long long P, int K)
{
    if (CK < 1 || CK > kThinFwdMaxCK || P % 4 != 0 || P < 64 || K < 1 || B < 1) return false;
    if (!aligned16(cols) || !aligned16(y)) return false;
    const long long quads = (long long)B * (P / 4), blocks = (quads + 255) / 256, groups = (K + kThinFwdGroup - 1) / kThinFwdGroup;
    if (blocks > kMaxGridX || groups > 65535) return false;
    hipLaunchKernelGGL(thin_fwd_kernel, dim3((unsigned)blocks, (unsigned)groups), dim3(256), 0, st, cols, w, y, (int)CK,
                       (int)(P / 4), K, quads);
    return true;
}

}  // namespace ag

extern "C" ag_status_t ag_conv2d_fwd_f32(ag_stream_t stream, const float *x, const float *w, float *y,
                                         float *cols, int B, int C, int H, int W, int K, int kh, int kw,
                                         int pad, int stride, int dilation)
{
    if (ag_status_t s = conv_dims("conv2d", B, C, H, W, K, kh, kw, pad, stride, dilation)) return s;
    AG_REQUIRE(H + 2 * pad >= dilation * (kh - 1) + 1 && W + 2 * pad >= dilation * (kw - 1) + 1,
               AG_ERR_INCOMPATIBLE_SHAPE, "conv2d: filter extent exceeds the padded input (%dx%d)", H, W);
    const int OH = ag_conv_out_size(H, kh, pad, stride, dilation);
    const int OW = ag_conv_out_size(W, kw, pad, stride, dilation);
    const long long CK = (long long)C * kh * kw, P = (long long)OH * OW;
    AG_REQUIRE(CK <= 0x7fffffff && P <= 0x7fffffff, AG_ERR_INVALID_DIMS, "conv2d: matrix extent overflows int");
    if (ag_status_t s = ag_im2col_f32(stream, x, cols, B, C, H, W, kh, kw, pad, pad, stride, stride, dilation,
                                      dilation))
        return s;
    if (w && y && cols && ag::thin_fwd(as_stream(stream), cols, w, y, B, CK, P, K)) return check_launch("conv2d");
    return ag_gemm_f32(stream, 0, 0, K, (int)P, (int)CK, 1.f, w, (int)CK, 0, cols, (int)P, CK * P, 0.f, y,
                       (int)P, (long long)K * P, B);
}

extern "C" ag_status_t ag_conv2d_with_cols_f32(ag_stream_t stream, const float *cols, const float *w,
                                               float *y, int B, int CK, int P, int K)
{
    if (w && y && cols && B >= 0 && CK >= 0 && P >= 0 && K >= 0 && ag::thin_fwd(as_stream(stream), cols, w, y, B, CK, P, K))
        return check_launch("conv2d_with_cols");
    return ag_gemm_f32(stream, 0, 0, K, P, CK, 1.f, w, CK, 0, cols, P, (long long)CK * P, 0.f, y, P,
                       (long long)K * P, B);
}

namespace ag {

// Filter gradient of a thin first layer (few filters, C*kh*kw of a few dozen at most, e.g. the
// 1 -> 32 channel 3x3 convolution of the small CNN): the output is a few hundred numbers summed
// over every position of every image, which leaves a tiled GEMM with one or two tiles per image.
// Here a block takes chunks of 128 positions, stages the K x 128 and CK x 128 operand slices in LDS
// (odd pitch: conflict-free) and every thread accumulates up to eight of the K*CK outputs over all
// the chunks of the block; one partial result per block, folded in block order by a second kernel.
constexpr int kThinChunk = 128, kThinPitch = kThinChunk + 1, kThinMaxK = 64, kThinMaxCK = 32, kThinMaxBlocks = 512;

__global__ __launch_bounds__(256) void thin_filter_grad_kernel(const float *__restrict__ cols, const float *__restrict__ gy,
                                                               float *__restrict__ partial, int B, int CK, int P, int K,
                                                               int chunks, long long items)
{
    __shared__ float s_gy[kThinMaxK * kThinPitch];
    __shared__ float s_co[kThinMaxCK * kThinPitch];
    const int outputs = K * CK;
    float acc[8] = {};
    for (long long item = blockIdx.x; item < items; item += gridDim.x) {
        const long long b = item / chunks;
        const int p0 = (int)(item - b * chunks) * kThinChunk, np = min(kThinChunk, P - p0);
        const float *gyb = gy + (b * K) * (long long)P + p0, *cob = cols + (b * CK) * (long long)P + p0;
        // thread -> position c of the chunk and every second row; all loads are issued before the
        // first LDS write, so their latencies overlap
        const int c = threadIdx.x & (kThinChunk - 1), rg = threadIdx.x >> 7;
        const bool in = c < np;
        float vg[kThinMaxK / 2], vc[kThinMaxCK / 2];
#pragma unroll
        for (int j = 0; j < kThinMaxK / 2; ++j) {
            const int r = rg + 2 * j;
            vg[j] = (in && r < K) ? gyb[(long long)r * P + c] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < kThinMaxCK / 2; ++j) {
            const int r = rg + 2 * j;
            vc[j] = (in && r < CK) ? cob[(long long)r * P + c] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < kThinMaxK / 2; ++j)
            if (rg + 2 * j < K) s_gy[(rg + 2 * j) * kThinPitch + c] = vg[j];
#pragma unroll
        for (int j = 0; j < kThinMaxCK / 2; ++j)
            if (rg + 2 * j < CK) s_co[(rg + 2 * j) * kThinPitch + c] = vc[j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int o = threadIdx.x + j * 256;
            if (o < outputs) {
                const float *a = s_gy + (o / CK) * kThinPitch, *c = s_co + (o % CK) * kThinPitch;
                // eight independent chains: the LDS reads of one do not wait for the adds of another
                float part[8] = {};
#pragma unroll 2
                for (int q = 0; q < kThinChunk; q += 8)
#pragma unroll
                    for (int u = 0; u < 8; ++u) part[u] += a[q + u] * c[q + u];
                acc[j] += ((part[0] + part[1]) + (part[2] + part[3])) + ((part[4] + part[5]) + (part[6] + part[7]));
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int o = threadIdx.x + j * 256;
        if (o < outputs) partial[(long long)blockIdx.x * outputs + o] = acc[j];
    }
}

// 32 outputs per block; eight groups of threads each add every eighth partial result (eight loads
// in flight), then the group sums are added in group order: a fixed order, so deterministic.
__global__ __launch_bounds__(256) void thin_filter_grad_fold_kernel(const float *__restrict__ partial, float *__restrict__ gw,
                                                                    int outputs, int blocks)
{
    __shared__ float part[8][32];
    const int oi = threadIdx.x & 31, grp = threadIdx.x >> 5;
    const int o = blockIdx.x * 32 + oi;
    float sum = 0.f;
    if (o < outputs) {
        int b = grp;
        for (; b + 56 < blocks; b += 64) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = partial[(long long)(b + 8 * u) * outputs + o];
#pragma unroll
            for (int u = 0; u < 8; ++u) sum += v[u];
        }
        for (; b < blocks; b += 8) sum += partial[(long long)b * outputs + o];
    }
    part[grp][oi] = sum;
    __syncthreads();
    if (grp == 0 && o < outputs) {
        float total = part[0][oi];
#pragma unroll
        for (int g2 = 1; g2 < 8; ++g2) total += part[g2][oi];
        gw[o] = total;
    }
}

static bool thin_filter_grad(int B, int CK, int P, int K)
{
    return K >= 1 && K <= kThinMaxK && CK >= 1 && CK <= kThinMaxCK && K * CK <= 2048 && P >= 64 && B >= 1;
}

static long long thin_blocks(int B, int P)
{
    const long long items = (long long)B * ((P + kThinChunk - 1) / kThinChunk);
    return items < kThinMaxBlocks ? items : kThinMaxBlocks;
}

}  // namespace ag

extern "C" size_t ag_conv2d_filter_grad_f32_workspace(int B, int CK, int P, int K)
{
    // (also the workspace of ag_conv2d_transpose_filter_grad_f32, which always runs the GEMM)
    const size_t gemm = ag_gemm_batchsum_f32_workspace(K, CK, P, B);
    const size_t thin = ag::thin_filter_grad(B, CK, P, K) ? sizeof(float) * (size_t)ag::thin_blocks(B, P) * K * CK : 0;
    return thin > gemm ? thin : gemm;
}

extern "C" ag_status_t ag_conv2d_filter_grad_f32(ag_stream_t stream, const float *cols, const float *gy,
                                                 float *gw, int B, int CK, int P, int K, void *ws,
                                                 size_t ws_bytes)
{
    // gw[K x CK] = sum_b gy_b[K x P] * cols_b[CK x P]^T        conv2d.rs:662-687
    if (ag::thin_filter_grad(B, CK, P, K)) {
        const long long blocks = ag::thin_blocks(B, P);
        const size_t need = sizeof(float) * (size_t)blocks * K * CK;
        AG_REQUIRE(cols && gy && gw, AG_ERR_INVALID_DIMS, "conv2d_filter_grad: null pointer");
        AG_REQUIRE(ws && ws_bytes >= need, AG_ERR_INVALID_DIMS, "conv2d_filter_grad: workspace of %zu bytes needed, %zu given",
                   need, ws_bytes);
        const int chunks = (P + ag::kThinChunk - 1) / ag::kThinChunk;
        hipLaunchKernelGGL(ag::thin_filter_grad_kernel, dim3((unsigned)blocks), dim3(256), 0, ag::as_stream(stream), cols, gy,
                           static_cast<float *>(ws), B, CK, P, K, chunks, (long long)B * chunks);
        hipLaunchKernelGGL(ag::thin_filter_grad_fold_kernel, dim3((unsigned)((K * CK + 31) / 32)), dim3(256), 0,
                           ag::as_stream(stream), static_cast<const float *>(ws), gw, K * CK, (int)blocks);
        return ag::check_launch("conv2d_filter_grad");
    }
    return ag_gemm_batchsum_f32(stream, 0, 1, K, CK, P, 1.f, gy, P, (long long)K * P, cols, P,
                                (long long)CK * P, 0.f, gw, CK, B, ws, ws_bytes);
}

namespace ag {


// gyp[plane][r][s] = gy[plane][r - top][s - left] inside the image, 0 in the border; four
// consecutive elements of the flattened padded plane per thread (its extent is a multiple of 4).
__global__ __launch_bounds__(256) void pad_border_kernel(const float *__restrict__ gy, float *__restrict__ gyp,
                                                         long long quads, int OH, int OW, int Hp, int Wp, int top,
                                                         int left)
{
    const unsigned plane_quads = (unsigned)(Hp * Wp) / 4u;
    for (long long qd = blockIdx.x * 256LL + threadIdx.x; qd < quads; qd += gridDim.x * 256LL) {
        // one division for the plane, one for the row; (row, column) then step along the four elements
        const long long plane = quads <= 0xffffffffLL ? (long long)((unsigned)qd / plane_quads) : qd / plane_quads;
        const unsigned e0 = (unsigned)(qd - plane * plane_quads) * 4u;
        int r = (int)(e0 / (unsigned)Wp), sx = (int)(e0 - (unsigned)r * (unsigned)Wp);
        const float *src = gy + plane * (long long)OH * OW;
        float v[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int oy = r - top, ox = sx - left;
            v[t] = ((unsigned)oy < (unsigned)OH && (unsigned)ox < (unsigned)OW) ? src[oy * OW + ox] : 0.f;
            if (++sx == Wp) {
                sx = 0;
                ++r;
            }
        }
        st_stream(reinterpret_cast<float4 *>(gyp) + qd, make_float4(v[0], v[1], v[2], v[3]));
    }
}

// wr[c][tap][k] = w[k][c][tap]  (tap = ky*kw + kx): the filter as the k-contiguous left operand of
// the implicit input-gradient GEMM.  Element e of wr.
__device__ inline float filter_tap(const float *__restrict__ w, int e, int Kf, int C, int taps)
{
    const int k = e % Kf, tap = e / Kf % taps, c = e / (Kf * taps);
    return w[((long long)k * C + c) * taps + tap];
}

// wf[k][tap'][c] = w[k][c][taps - 1 - tap']: the filter as the left operand of the implicit forward
// GEMM.  The GEMM visits its taps from the largest shift to none (the order the input gradient
// needs), so a correlation lists them reversed.  Element e of wf.
__device__ inline float filter_tap_fwd(const float *__restrict__ w, int e, int C, int taps)
{
    const int c = e % C, tap = e / C % taps, k = e / (C * taps);
    return w[((long long)k * C + c) * taps + (taps - 1 - tap)];
}

// Four floats at an address that is only 4-byte aligned.
struct __attribute__((packed, aligned(4))) Unaligned4 {
    float x, y, z, w;
};

// The small jobs that accompany a bordered copy (see pad_border_fast_kernel).
struct PrepareExtras {
    float *lead;     // n_lead floats to zero before the planes
    int n_lead;
    float *tail;     // n_tail floats to zero after them
    int n_tail;
    const float *w;  // filter [Kf][C][taps] ...
    float *wt;       // ... rewritten here (nullptr: not asked for)
    int Kf, C, taps;
    int fwd;         // 1: forward order (filter_tap_fwd), 0: input-gradient order (filter_tap)
};

// The same copy with the divisions replaced by multiplications: grid.y walks the images, so the
// element counter stays small enough for n / d == umulhi(n, floor(2^32 / d) + 1) to be exact (the
// host checks the range).  gyp [B][planes][Hp][Wp]; quads_img = planes * Hp * Wp / 4.
// The same launch does the two small jobs that go with every bordered copy -- zeroing the slack around the planes
// and writing the filter in the tap order of the implicit GEMM -- so that preparing an operand is one launch.  They
// are dealt out over the threads of the whole grid, one element (or a few) each: the filter is gathered at a
// stride of a whole filter row, a load per element that waits out the memory latency, and 590 k elements (256 ->
// 256 channels, 3 x 3) in the hands of one grid row of 72 blocks took 15 us where the copy itself takes 5.
__global__ __launch_bounds__(256) void pad_border_fast_kernel(const float *__restrict__ gy, float *__restrict__ gyp,
                                                              unsigned quads_img, unsigned planes, int OH, int OW, int Wp,
                                                              int top, int left, unsigned plane_quads, unsigned m_plane,
                                                              unsigned m_row, int B, PrepareExtras ex)
{
    const unsigned ny = gridDim.y;
    {
        const long long gt = ((long long)blockIdx.y * gridDim.x + blockIdx.x) * 256 + threadIdx.x;
        const int slack = ex.n_lead + ex.n_tail, total = slack + (ex.wt ? ex.Kf * ex.C * ex.taps : 0);
        if (gt < total) {
            const long long nth = (long long)gridDim.x * gridDim.y * 256;
            for (long long i = gt; i < total; i += nth) {
                if (i < ex.n_lead) ex.lead[i] = 0.f;
                else if (i < slack) ex.tail[i - ex.n_lead] = 0.f;
                else ex.wt[i - slack] = ex.fwd ? filter_tap_fwd(ex.w, (int)(i - slack), ex.C, ex.taps)
                                               : filter_tap(ex.w, (int)(i - slack), ex.Kf, ex.C, ex.taps);
            }
        }
    }
    const unsigned qi = blockIdx.x * 256u + threadIdx.x;
    if (qi >= quads_img) return;
    const unsigned pl = __umulhi(qi, m_plane);
    const unsigned e0 = (qi - pl * plane_quads) * 4u;
    int r = (int)__umulhi(e0, m_row), sx = (int)(e0 - (unsigned)r * (unsigned)Wp);
    // (row, column) of the four elements relative to the image data
    int oy[4], ox[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        oy[t] = r - top;
        ox[t] = sx - left;
        if (++sx == Wp) {
            sx = 0;
            ++r;
        }
    }
    // Four elements that lie side by side inside one row of the image are one 16-byte load (aligned to 4 bytes only: the
    // border shifts the copy against the source); the quads that touch a border or run over a row's end load what
    // they have of the image one element at a time.
    const bool whole = oy[3] == oy[0] && (unsigned)oy[0] < (unsigned)OH && ox[0] >= 0 && ox[3] < OW;
    const int first = oy[0] * OW + ox[0];
    for (int b = blockIdx.y; b < B; b += ny) {
        const float *src = gy + ((long long)b * planes + pl) * (long long)OH * OW;
        float v[4];
        if (whole) {
            const Unaligned4 q = *reinterpret_cast<const Unaligned4 *>(src + first);
            v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
        } else {
#pragma unroll
            for (int t = 0; t < 4; ++t)
                v[t] = ((unsigned)oy[t] < (unsigned)OH && (unsigned)ox[t] < (unsigned)OW) ? src[oy[t] * OW + ox[t]] : 0.f;
        }
        st_stream(reinterpret_cast<float4 *>(gyp) + ((long long)b * quads_img + qi), make_float4(v[0], v[1], v[2], v[3]));
    }
}

// Launches the bordered copy of `planes` planes per image.  With `extras` the same launch also zeroes the slack
// and rewrites the filter when it can (returns true); otherwise the caller launches those itself.
static bool launch_pad_border_with(hipStream_t st, const float *src, float *dst, int B, int planes, int OH, int OW, int Hp,
                                   int Wp, int top, int left, const PrepareExtras *extras)
{
    const long long plane_quads = (long long)Hp * Wp / 4, quads_img = plane_quads * planes;
    // exactness of the two multiply-high divisions: n * (m * d - 2^32) < 2^32 with m * d - 2^32 <= d
    const bool fast = quads_img * plane_quads < (1LL << 32) && (long long)Hp * Wp * Wp < (1LL << 32) && plane_quads > 1 && Wp > 1;
    if (fast) {
        const unsigned m_plane = (unsigned)((1ULL << 32) / (unsigned long long)plane_quads) + 1u;
        const unsigned m_row = (unsigned)((1ULL << 32) / (unsigned long long)Wp) + 1u;
        // one grid row per image (at most 65534)
        const dim3 grid((unsigned)((quads_img + 255) / 256), (unsigned)(B < 65534 ? B : 65534));
        const bool fits = extras && (!extras->wt || (long long)extras->Kf * extras->C * extras->taps < 0x7ffff000LL);
        PrepareExtras ex = {};
        if (fits) ex = *extras;
        hipLaunchKernelGGL(pad_border_fast_kernel, grid, dim3(256), 0, st, src, dst, (unsigned)quads_img, (unsigned)planes, OH, OW,
                           Wp, top, left, (unsigned)plane_quads, m_plane, m_row, B, ex);
        return fits;
    }
    const long long quads = quads_img * B;
    long long blocks = (quads + 255) / 256;
    if (blocks > 1048576) blocks = 1048576;
    hipLaunchKernelGGL(pad_border_kernel, dim3((unsigned)blocks), dim3(256), 0, st, src, dst, quads, OH, OW, Hp, Wp, top, left);
    return false;
}

void launch_pad_border(hipStream_t st, const float *src, float *dst, int B, int planes, int OH, int OW, int Hp, int Wp,
                       int top, int left)
{
    launch_pad_border_with(st, src, dst, B, planes, OH, OW, Hp, Wp, top, left, nullptr);
}

// Zeroes the slack before and after the padded planes: the implicit filter gradient multiplies what
// it reads there by border zeros of the gradient, which must not meet a NaN bit pattern.
__global__ void zero_slack_kernel(float *lead, int n_lead, float *tail, int n_tail)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n_lead + n_tail; i += gridDim.x * blockDim.x) {
        if (i < n_lead) lead[i] = 0.f;
        else tail[i - n_lead] = 0.f;
    }
}

// The filter in input-gradient order (filter_tap) as a launch of its own.
__global__ __launch_bounds__(256) void filter_taps_kernel(const float *__restrict__ w, float *__restrict__ wr, int Kf,
                                                          int C, int taps)
{
    const int total = Kf * C * taps;
    for (int e = blockIdx.x * 256 + threadIdx.x; e < total; e += gridDim.x * 256) wr[e] = filter_tap(w, e, Kf, C, taps);
}

// The filter in forward order (filter_tap_fwd) as a launch of its own.
__global__ __launch_bounds__(256) void filter_taps_fwd_kernel(const float *__restrict__ w, float *__restrict__ wf, int Kf,
                                                              int C, int taps)
{
    const int total = Kf * C * taps;
    for (int e = blockIdx.x * 256 + threadIdx.x; e < total; e += gridDim.x * 256) wf[e] = filter_tap_fwd(w, e, C, taps);
}

// Zeroed floats after the last bordered plane (and before the first one of a bordered input).
constexpr long long kSlackFloats = 1024;

// Geometry of the implicit (column-free) stride-1 input gradient.
struct FusedGeom {
    int Hp, Wp;
    long long gyp_floats, wr_floats;  // scratch layout: zero-bordered gy, then the tap-major filter,
    long long ws_floats;              // then the partial results of a split contraction (0: none)
};

// False when the geometry does not allow the implicit path.
// `dil`: the filter taps are dil apart; borders and reach follow the filter's extent ekh = dil*(kh-1)+1.
static bool fused_geom(int B, int ych, int yh, int yw, int xch, int kh, int kw, int pad, int xh, int xw, FusedGeom *g, int dil = 1)
{
    const int ekh = dil * (kh - 1) + 1, ekw = dil * (kw - 1) + 1;
    if (dil < 1 || pad > ekh - 1 || pad > ekw - 1 || ych % 32 != 0 || B < 1 || xch < 1) return false;
    if (yh != xh + 2 * pad - ekh + 1 || yw != xw + 2 * pad - ekw + 1 || yh < 1 || yw < 1) return false;
    // A padded row holds the left border (kw-1-pad zeros) and the data; it needs no right border of
    // its own: a read that runs past the end of a row by up to kw-1-pad elements lands in the left
    // border of the next row, which is just as zero.  The row pitch and the plane (rows added at the
    // bottom) grow until the per-image column range and the plane are multiples of four elements.
    // The implicit filter gradient contracts over the positions of a plane rounded up to its k tile
    // (32) and reads the other operand up to kh-1 rows and kw-1 elements further: rows are added until
    // everything it reads past a plane's own data is zero -- the rows below the data, then the top
    // border of the next plane up to the first data element of its first data row -- so that no value
    // of a neighbouring plane (which could be a NaN) ever meets one of those zeros.  A plane plays one of two
    // parts there: as the gradient it is read from its first data element on (border `top`), as the input it is
    // read from its origin on but up to a filter's reach further, which comes to the same bound with the border
    // of the other part (`pad`): the larger of the two sizes the plane.
    const int top = ekh - 1 - pad, left = ekw - 1 - pad;
    const int guard_t = top > pad ? top : pad, guard_l = left > pad ? left : pad;
    g->Wp = yw + left;
    for (;; ++g->Wp) {
        if (g->Wp > xw + ekw + 6) return false;
        // (the rows of this tensor and of the one it is contracted into: the bordered copies of x and of gy then
        // come out with one row pitch, which the implicit filter gradient needs)
        if (((long long)xh * g->Wp) % 4 != 0 || ((long long)yh * g->Wp) % 4 != 0) continue;
        g->Hp = xh + ekh - 1;
        const long long kq = (((long long)xh * g->Wp + 31) / 32) * 32;
        while (((long long)g->Hp * g->Wp) % 4 != 0 || (long long)(g->Hp - guard_t) * g->Wp - guard_l < kq) ++g->Hp;
        break;
    }
    // past the last plane the reads run into kSlackFloats zeroed floats
    if ((long long)(ekh - 1) * g->Wp + 2 * (ekw - 1) + 32 > kSlackFloats) return false;
    const long long plane = (long long)g->Hp * g->Wp, n_img = (long long)xh * g->Wp;
    g->gyp_floats = (long long)B * ych * plane + kSlackFloats;  // slack: the last taps read a little past a plane
    g->wr_floats = (long long)xch * kh * kw * ych;
    g->ws_floats = (long long)gemm_conv_input_grad_ws_floats(B, xch, ych, xh, xw, g->Wp, kh * kw);
    // a tile may cover any number of images; the loader's 32-bit byte offsets reach over a k tile's 32 planes and as many
    // images further as a tile of up to 256 columns can run into
    const long long more_imgs = n_img >= 256 ? 1 : 256 / n_img + 1;
    if (32 * plane + more_imgs * ych * plane >= (1LL << 30)) return false;
    return n_img >= 16 && B * n_img < 0x7fffffffLL && ych * plane < (1LL << 30);
}

static ag_status_t fused_prepare(hipStream_t st, const float *gy, const float *w, float *scratch, const FusedGeom &g,
                                 int B, int ych, int yh, int yw, int xch, int kh, int kw, int pad, int dil = 1)
{
    const long long quads = (long long)B * ych * g.Hp * g.Wp / 4;
    // the implicit filter gradient may read a few elements past the last plane and expects zeros
    const PrepareExtras ex = {scratch, 0, scratch + quads * 4, (int)(g.gyp_floats - quads * 4), w, scratch + g.gyp_floats,
                              ych, xch, kh * kw, 0};
    if (!launch_pad_border_with(st, gy, scratch, B, ych, yh, yw, g.Hp, g.Wp, dil * (kh - 1) - pad, dil * (kw - 1) - pad, &ex)) {
        hipLaunchKernelGGL(zero_slack_kernel, dim3(4), dim3(256), 0, st, ex.lead, ex.n_lead, ex.tail, ex.n_tail);
        hipLaunchKernelGGL(filter_taps_kernel, dim3((unsigned)((g.wr_floats + 255) / 256)), dim3(256), 0, st, w,
                           scratch + g.gyp_floats, ych, xch, kh * kw);
    }
    return check_launch("conv2d_transpose");
}

// The column-free forward is the same implicit GEMM with the roles exchanged: the input x takes the
// place of the upstream gradient (bordered by `pad`), the C input channels are contracted and the K
// filters are the output rows.  Leading slack: the implicit filter gradient reads up to one padded
// row and column before the first plane.
constexpr long long kFwdLeadFloats = kSlackFloats;

static bool fused_fwd_geom(int B, int C, int H, int W, int K, int kh, int kw, int pad, FusedGeom *g, int dil = 1)
{
    const int ekh = dil * (kh - 1) + 1, ekw = dil * (kw - 1) + 1;
    const int OH = H + 2 * pad - ekh + 1, OW = W + 2 * pad - ekw + 1;
    if (dil < 1 || OH < 1 || OW < 1 || pad > ekh - 1 || pad > ekw - 1) return false;
    // seen as an input gradient: "gy" = x [C, H, W], "gx" = y [K, OH, OW], border ekh-1-pad' = pad
    return kh == kw && fused_geom(B, C, H, W, K, kh, kw, ekh - 1 - pad, OH, OW, g, dil);
}

// Positions of the flattened padded plane that the implicit filter gradient contracts over: all
// rows that hold gradient values, rounded up to the GEMM's k tile.  0 = the rounding would reach
// past zeros.
// `gx`: the bordered input (border pad), `gg`: the bordered gradient (border reach - pad, reach = dil * (k - 1)).
static int filter_grad_positions(const FusedGeom &gx, const FusedGeom &gg, int OH, int pad, int reach)
{
    // The gradient is read from its first value on: what follows its OH rows must be zeros up to position kq (its
    // bottom rows, then the next plane's top border or the zeroed slack).  The input is read from its origin on,
    // up to `reach` rows and elements past position kq: that may run into the next plane's top border (pad rows and
    // elements of zeros) but not into its data.  Both come to the same bound; fused_geom sizes the planes for it.
    const long long kq = (((long long)OH * gx.Wp + 31) / 32) * 32;
    const int b = reach - pad;
    if (gx.Wp != gg.Wp || b < 0) return 0;
    const bool ok = kq <= (long long)(gx.Hp - b) * gx.Wp - b && kq <= (long long)(gg.Hp - b) * gg.Wp - b;
    return ok ? (int)kq : 0;
}

}  // namespace ag

// ---- column-free convolution: forward and filter gradient ---------------------------------------
// No counterpart of these in the reference, which always materialises the columns
// (conv2d.rs:25-112, 631-734); they compute the same y and gw from a rearranged copy of x: the
// zero-bordered input for stride 1 (any dilation), its four phase planes for stride 2 (conv_s2.hip; dilation
// 1 only).  `xpad`: ag_conv2d_nocols_scratch_floats() floats, written by the forward and read by the
// filter gradient.  0 floats = geometry not supported (use ag_conv2d_fwd_f32 / ag_conv2d_filter_grad_f32).
namespace ag {
static bool nocols_mode(int stride, int dilation) { return (stride == 1 && dilation >= 1) || (stride == 2 && dilation == 1); }
}  // namespace ag

extern "C" size_t ag_conv2d_nocols_scratch_floats(int B, int C, int H, int W, int K, int kh, int kw, int pad, int stride,
                                                  int dilation)
{
    if (!nocols_mode(stride, dilation)) return 0;
    if (stride == 2) {
        S2Geom g2;
        return s2_geom(B, C, H, W, K, kh, kw, pad, &g2) ? (size_t)(g2.xph_floats + g2.wf_floats) : 0;
    }
    FusedGeom g;
    if (!fused_fwd_geom(B, C, H, W, K, kh, kw, pad, &g, dilation)) return 0;
    return (size_t)(kFwdLeadFloats + g.gyp_floats + g.wr_floats + g.ws_floats);
}

// The two stages of the forward, for callers that time or schedule them separately.
extern "C" ag_status_t ag_conv2d_nocols_prepare_f32(ag_stream_t stream, const float *x, const float *w, float *xpad, int B,
                                                    int C, int H, int W, int K, int kh, int kw, int pad, int stride, int dilation)
{
    AG_REQUIRE(nocols_mode(stride, dilation), AG_ERR_INVALID_DIMS, "conv2d (column-free): stride %d / dilation %d not supported",
               stride, dilation);
    AG_REQUIRE(x && w && xpad, AG_ERR_INVALID_DIMS, "conv2d (column-free): null pointer");
    hipStream_t st = as_stream(stream);
    if (stride == 2) {
        S2Geom g2;
        AG_REQUIRE(s2_geom(B, C, H, W, K, kh, kw, pad, &g2) && aligned16(xpad), AG_ERR_INVALID_DIMS,
                   "conv2d (column-free): geometry not supported");
        return s2_fwd_prepare(st, x, w, xpad, g2, B, C, H, W, K, kh, kw, pad);
    }
    FusedGeom g;
    AG_REQUIRE(fused_fwd_geom(B, C, H, W, K, kh, kw, pad, &g, dilation) && aligned16(xpad), AG_ERR_INVALID_DIMS,
               "conv2d (column-free): geometry not supported");
    float *xp = xpad + kFwdLeadFloats, *wf = xp + g.gyp_floats;
    const long long quads = (long long)B * C * g.Hp * g.Wp / 4;
    const PrepareExtras ex = {xpad, (int)kFwdLeadFloats, xp + quads * 4, (int)(g.gyp_floats - quads * 4), w, wf, K, C, kh * kw, 1};
    if (!launch_pad_border_with(st, x, xp, B, C, H, W, g.Hp, g.Wp, pad, pad, &ex)) {
        hipLaunchKernelGGL(zero_slack_kernel, dim3(8), dim3(256), 0, st, ex.lead, ex.n_lead, ex.tail, ex.n_tail);
        hipLaunchKernelGGL(filter_taps_fwd_kernel, dim3((unsigned)((g.wr_floats + 255) / 256)), dim3(256), 0, st, w, wf, K, C,
                           kh * kw);
    }
    return check_launch("conv2d");
}

extern "C" ag_status_t ag_conv2d_nocols_gemm_f32(ag_stream_t stream, float *xpad, float *y, int B, int C, int H, int W,
                                                 int K, int kh, int kw, int pad, int stride, int dilation)
{
    AG_REQUIRE(nocols_mode(stride, dilation), AG_ERR_INVALID_DIMS, "conv2d (column-free): stride %d / dilation %d not supported",
               stride, dilation);
    AG_REQUIRE(xpad && y, AG_ERR_INVALID_DIMS, "conv2d (column-free): null pointer");
    if (stride == 2) {
        S2Geom g2;
        AG_REQUIRE(s2_geom(B, C, H, W, K, kh, kw, pad, &g2) && aligned16(xpad) && aligned16(y), AG_ERR_INVALID_DIMS,
                   "conv2d (column-free): geometry not supported");
        return s2_fwd_gemm(as_stream(stream), xpad, xpad + g2.xph_floats, y, g2, B, C, K, kh, kw);
    }
    FusedGeom g;
    AG_REQUIRE(fused_fwd_geom(B, C, H, W, K, kh, kw, pad, &g, dilation) && aligned16(xpad) && aligned16(y), AG_ERR_INVALID_DIMS,
               "conv2d (column-free): geometry not supported");
    float *xp = xpad + kFwdLeadFloats;
    float *ws = xp + g.gyp_floats + g.wr_floats;  // (the part of xpad behind the filter: partial results, transient)
    return gemm_conv_input_grad(as_stream(stream), xp + g.gyp_floats, xp, y, B, K, C, H + 2 * pad - dilation * (kh - 1),
                                W + 2 * pad - dilation * (kw - 1), kh, kw, g.Hp, g.Wp, dilation, g.ws_floats ? ws : nullptr,
                                (size_t)g.ws_floats);
}

extern "C" ag_status_t ag_conv2d_fwd_nocols_f32(ag_stream_t stream, const float *x, const float *w, float *y, float *xpad,
                                                int B, int C, int H, int W, int K, int kh, int kw, int pad, int stride,
                                                int dilation)
{
    if (ag_status_t s = ag_conv2d_nocols_prepare_f32(stream, x, w, xpad, B, C, H, W, K, kh, kw, pad, stride, dilation)) return s;
    return ag_conv2d_nocols_gemm_f32(stream, xpad, y, B, C, H, W, K, kh, kw, pad, stride, dilation);
}

// The forward GEMM over an existing rearranged copy with another filter (Conv2DWithCols, conv2d.rs:
// 589-629, when the "columns" it is given are such a copy): `wf` receives K*C*kh*kw floats.
extern "C" ag_status_t ag_conv2d_nocols_with_filter_f32(ag_stream_t stream, const float *xpad, const float *w, float *wf,
                                                        float *y, int B, int C, int H, int W, int K, int kh, int kw, int pad,
                                                        int stride, int dilation)
{
    AG_REQUIRE(nocols_mode(stride, dilation), AG_ERR_INVALID_DIMS, "conv2d (column-free): stride %d / dilation %d not supported",
               stride, dilation);
    AG_REQUIRE(xpad && w && wf && y, AG_ERR_INVALID_DIMS, "conv2d (column-free): null pointer");
    hipStream_t st = as_stream(stream);
    if (stride == 2) {
        S2Geom g2;
        AG_REQUIRE(s2_geom(B, C, H, W, K, kh, kw, pad, &g2) && aligned16(xpad) && aligned16(y) && aligned16(wf), AG_ERR_INVALID_DIMS,
                   "conv2d (column-free): geometry not supported");
        if (ag_status_t s = s2_fwd_filter(st, w, wf, g2, C, K, kh, kw)) return s;
        return s2_fwd_gemm(st, xpad, wf, y, g2, B, C, K, kh, kw);
    }
    FusedGeom g;
    AG_REQUIRE(fused_fwd_geom(B, C, H, W, K, kh, kw, pad, &g, dilation) && aligned16(xpad) && aligned16(y) && aligned16(wf),
               AG_ERR_INVALID_DIMS, "conv2d (column-free): geometry not supported");
    hipLaunchKernelGGL(filter_taps_fwd_kernel, dim3((unsigned)((g.wr_floats + 255) / 256)), dim3(256), 0, st, w, wf, K, C,
                       kh * kw);
    if (ag_status_t s = check_launch("conv2d")) return s;
    return gemm_conv_input_grad(st, wf, xpad + kFwdLeadFloats, y, B, K, C, H + 2 * pad - dilation * (kh - 1),
                                W + 2 * pad - dilation * (kw - 1), kh, kw, g.Hp, g.Wp, dilation);
}

// gypad: the zero-bordered upstream gradient written by ag_conv_input_grad_prepare_f32 (the start
// of its scratch).  Stride 1: x' carries a border of pad, gy' one of reach - pad (reach = dilation * (k - 1)); both
// have the row pitch W + pad (rounded alike), so a position of the flattened gy' plane and the same position of the
// x' plane shifted by a tap are the two factors of one product.  Their plane heights differ unless 2 * pad == reach.
extern "C" size_t ag_conv2d_filter_grad_nocols_f32_workspace(int B, int C, int H, int W, int K, int kh, int kw, int pad,
                                                             int stride, int dilation)
{
    if (!nocols_mode(stride, dilation)) return 0;
    if (stride == 2) {
        S2Geom g2;
        return s2_geom(B, C, H, W, K, kh, kw, pad, &g2) ? s2_filter_grad_workspace(g2, B, C, K, kh, kw) : 0;
    }
    FusedGeom g, gg;
    const int OH = H + 2 * pad - dilation * (kh - 1), OW = W + 2 * pad - dilation * (kw - 1);
    if (K % 4 != 0 || !fused_fwd_geom(B, C, H, W, K, kh, kw, pad, &g, dilation) ||
        !fused_geom(B, K, OH, OW, C, kh, kw, pad, H, W, &gg, dilation) || (long long)C * g.Hp * g.Wp >= (1LL << 30) ||
        (long long)K * gg.Hp * gg.Wp >= (1LL << 30))
        return 0;
    const int kq = filter_grad_positions(g, gg, OH, pad, dilation * (kh - 1));
    return kq ? gemm_conv_filter_grad_workspace(B, K, C, kh * kw, kq) : 0;
}

extern "C" ag_status_t ag_conv2d_filter_grad_nocols_f32(ag_stream_t stream, const float *xpad, const float *gypad, float *gw,
                                                        int B, int C, int H, int W, int K, int kh, int kw, int pad, int stride,
                                                        int dilation, void *ws, size_t ws_bytes)
{
    AG_REQUIRE(nocols_mode(stride, dilation), AG_ERR_INVALID_DIMS,
               "conv2d_filter_grad (column-free): stride %d / dilation %d not supported", stride, dilation);
    AG_REQUIRE(gw, AG_ERR_INVALID_DIMS, "conv2d_filter_grad (column-free): null output");
    if (stride == 2) {
        S2Geom g2;
        AG_REQUIRE(s2_geom(B, C, H, W, K, kh, kw, pad, &g2) && aligned16(xpad) && aligned16(gypad), AG_ERR_INVALID_DIMS,
                   "conv2d_filter_grad (column-free): geometry not supported");
        return s2_filter_grad(as_stream(stream), xpad, gypad, gw, g2, B, C, K, kh, kw, ws, ws_bytes);
    }
    FusedGeom g, gg;
    const int OH = H + 2 * pad - dilation * (kh - 1), OW = W + 2 * pad - dilation * (kw - 1);
    AG_REQUIRE(K % 4 == 0 && C >= 1 && fused_fwd_geom(B, C, H, W, K, kh, kw, pad, &g, dilation) &&
                   fused_geom(B, K, OH, OW, C, kh, kw, pad, H, W, &gg, dilation) && aligned16(xpad) && aligned16(gypad),
               AG_ERR_INVALID_DIMS, "conv2d_filter_grad (column-free): geometry not supported");
    const int reach = dilation * (kh - 1);
    const int kq = filter_grad_positions(g, gg, OH, pad, reach);
    AG_REQUIRE(kq > 0 && (long long)C * g.Hp * g.Wp < (1LL << 30) && (long long)K * gg.Hp * gg.Wp < (1LL << 30), AG_ERR_INVALID_DIMS,
               "conv2d_filter_grad (column-free): the bordered planes of x and gy do not line up, or too many channels");
    return gemm_conv_filter_grad(as_stream(stream), gypad, xpad + kFwdLeadFloats, gw, ws, ws_bytes, B, K, C, kh, kw, reach - pad,
                                 gg.Hp, g.Hp, g.Wp, kq, dilation);
}

extern "C" ag_status_t ag_conv2d_transpose_f32(ag_stream_t stream, const float *gy, const float *w,
                                               float *gx, float *gcols, int B, int ych, int yh, int yw,
                                               int xch, int kh, int kw, int pad, int stride, int dilation,
                                               int xh, int xw)
{
    if (ag_status_t s = conv_dims("conv2d_transpose", B, xch, xh, xw, ych, kh, kw, pad, stride, dilation)) return s;
    AG_REQUIRE(yh >= 0 && yw >= 0, AG_ERR_INVALID_DIMS, "conv2d_transpose: negative extent (%dx%d)", yh, yw);
    const long long M = (long long)xch * kh * kw, P = (long long)yh * yw;
    AG_REQUIRE(M <= 0x7fffffff && P <= 0x7fffffff, AG_ERR_INVALID_DIMS,
               "conv2d_transpose: matrix extent overflows int");
    // every column position must map inside [-pad, x + pad): same geometry as the forward conv
    AG_REQUIRE(yh == 0 || yw == 0 ||
                   ((yh - 1) * stride + dilation * (kh - 1) + 1 <= xh + 2 * pad &&
                    (yw - 1) * stride + dilation * (kw - 1) + 1 <= xw + 2 * pad),
               AG_ERR_INCOMPATIBLE_SHAPE,
               "conv2d_transpose: output %dx%d too small for input %dx%d (k=%dx%d stride=%d pad=%d dilation=%d)", xh,
               xw, yh, yw, kh, kw, stride, pad, dilation);
    // Stride 1: the gradient is accumulated over filter taps inside one GEMM that
    // reads a zero-bordered copy of gy; the columns (conv2d_transpose.rs:148-151) are never
    // written.  The sum runs over (tap, filter) instead of filters then taps, within tolerance.
    FusedGeom fg;
    // (images of fewer than 256 padded positions with more than 64 channels run on 64-row tiles, and while their
    // columns stay in the cache the column path is ahead: 32 x 256 -> 256 channels, 14 x 14: 0.084 against 0.108 ms;
    // at eight times the batch 0.71 against 0.54 ms)
    if (stride == 1 &&
        fused_geom(B, ych, yh, yw, xch, kh, kw, pad, xh, xw, &fg, dilation) && fg.gyp_floats + fg.wr_floats <= (long long)B * M * P &&
        ((long long)xh * fg.Wp >= 256 || xch <= 64 || (long long)B * M * P >= (1LL << 24)) && aligned16(gcols) && aligned16(gx)) {
        if (ag_status_t s = fused_prepare(as_stream(stream), gy, w, gcols, fg, B, ych, yh, yw, xch, kh, kw, pad, dilation)) return s;
        // (what the column buffer has left behind the bordered gradient and the filter serves a split contraction)
        const bool room = fg.ws_floats > 0 && fg.gyp_floats + fg.wr_floats + fg.ws_floats <= (long long)B * M * P;
        return gemm_conv_input_grad(as_stream(stream), gcols + fg.gyp_floats, gcols, gx, B, xch, ych, xh, xw, kh, kw, fg.Hp,
                                    fg.Wp, dilation, room ? gcols + fg.gyp_floats + fg.wr_floats : nullptr,
                                    room ? (size_t)fg.ws_floats : 0);
    }
    // Stride 2: parity GEMMs over one bordered copy of gy (conv_s2.hip), when the columns' buffer
    // is large enough to serve as their scratch.  Only from 2^24 column elements on: below that the
    // launches and the short contractions cost more than GEMM + col2im (the 4x4 stride-2 transposed
    // convolution [32,128,14,14] -> [32,64,28,28] with both gradients takes 0.21 ms this way against
    // 0.13 ms over columns).
    S2Geom g2;
    if (stride == 2 && dilation == 1 && (long long)B * M * P >= (1LL << 24) &&
        s2_geom(B, xch, xh, xw, ych, kh, kw, pad, &g2) && g2.OH == yh &&
        g2.OW == yw && g2.gyp_floats + g2.wf_floats + g2.gxp_floats <= (long long)B * M * P && aligned16(gcols) && aligned16(gx)) {
        if (ag_status_t s = s2_igrad_prepare(as_stream(stream), gy, w, gcols, g2, B, xch, ych, kh, kw, pad)) return s;
        return s2_igrad_gemm(as_stream(stream), gcols, gx, g2, B, xch, ych, xh, xw);
    }
    // gcols_b[M x P] = w^T[M x ych] * gy_b[ych x P]               conv2d_transpose.rs:114-116,167-182
    if (ag_status_t s = ag_gemm_f32(stream, 1, 0, (int)M, (int)P, ych, 1.f, w, (int)M, 0, gy, (int)P,
                                    (long long)ych * P, 0.f, gcols, (int)P, M * P, B))
        return s;
    return ag_col2im_f32(stream, gcols, gx, B, xch, xh, xw, kh, kw, pad, pad, stride, stride, dilation, dilation,
                         yh, yw);
}

extern "C" ag_status_t ag_conv2d_transpose_filter_grad_f32(ag_stream_t stream, const float *x,
                                                           const float *gy, float *gw, float *gycols, int B,
                                                           int ych, int yh, int yw, int xch, int H, int W,
                                                           int kh, int kw, int pad, int stride, int dilation,
                                                           void *ws, size_t ws_bytes)
{
    if (ag_status_t s = conv_dims("conv2d_transpose_filter_grad", B, xch, H, W, ych, kh, kw, pad, stride, dilation))
        return s;
    AG_REQUIRE(H + 2 * pad >= dilation * (kh - 1) + 1 && W + 2 * pad >= dilation * (kw - 1) + 1,
               AG_ERR_INCOMPATIBLE_SHAPE, "conv2d_transpose_filter_grad: filter extent exceeds the padded gradient (%dx%d)",
               H, W);
    AG_REQUIRE(ag_conv_out_size(H, kh, pad, stride, dilation) == yh &&
                   ag_conv_out_size(W, kw, pad, stride, dilation) == yw,
               AG_ERR_INCOMPATIBLE_SHAPE,
               "conv2d_transpose_filter_grad: gradient %dx%d does not reduce to the input's %dx%d", H, W, yh, yw);
    const long long N = (long long)xch * kh * kw, P = (long long)yh * yw;
    AG_REQUIRE(N <= 0x7fffffff && P <= 0x7fffffff, AG_ERR_INVALID_DIMS,
               "conv2d_transpose_filter_grad: matrix extent overflows int");
    // gy -> columns                                              conv2d_transpose.rs:331-345
    if (ag_status_t s = ag_im2col_f32(stream, gy, gycols, B, xch, H, W, kh, kw, pad, pad, stride, stride, dilation,
                                      dilation))
        return s;
    // gw[ych x N] = sum_b x_b[ych x P] * gycols_b[N x P]^T        conv2d_transpose.rs:354-381
    return ag_gemm_batchsum_f32(stream, 0, 1, ych, (int)N, (int)P, 1.f, x, (int)P, (long long)ych * P, gycols,
                                (int)P, N * P, 0.f, gw, (int)N, B, ws, ws_bytes);
}

// The two stages of the column-free stride-1 input gradient, for callers that time or schedule
// them separately.  `scratch` holds ag_conv_input_grad_scratch_floats() floats (0 = this
// geometry takes the GEMM + col2im path and the staged entry points refuse it).
extern "C" size_t ag_conv_input_grad_scratch_floats(int B, int ych, int yh, int yw, int xch, int kh, int kw, int pad,
                                                    int stride, int dilation, int xh, int xw)
{
    if (!nocols_mode(stride, dilation)) return 0;
    if (stride == 2) {
        S2Geom g2;
        if (!s2_geom(B, xch, xh, xw, ych, kh, kw, pad, &g2) || g2.OH != yh || g2.OW != yw) return 0;
        return (size_t)(g2.gyp_floats + g2.wf_floats + g2.gxp_floats);
    }
    FusedGeom g;
    return fused_geom(B, ych, yh, yw, xch, kh, kw, pad, xh, xw, &g, dilation) ? (size_t)(g.gyp_floats + g.wr_floats + g.ws_floats) : 0;
}

extern "C" ag_status_t ag_conv_input_grad_prepare_f32(ag_stream_t stream, const float *gy, const float *w, float *scratch,
                                                      int B, int ych, int yh, int yw, int xch, int kh, int kw, int pad,
                                                      int stride, int dilation, int xh, int xw)
{
    AG_REQUIRE(nocols_mode(stride, dilation), AG_ERR_INVALID_DIMS, "conv_input_grad_prepare: stride %d / dilation %d not supported",
               stride, dilation);
    AG_REQUIRE(gy && w && scratch, AG_ERR_INVALID_DIMS, "conv_input_grad_prepare: null pointer");
    if (stride == 2) {
        S2Geom g2;
        AG_REQUIRE(s2_geom(B, xch, xh, xw, ych, kh, kw, pad, &g2) && g2.OH == yh && g2.OW == yw && aligned16(scratch),
                   AG_ERR_INVALID_DIMS, "conv_input_grad_prepare: geometry not supported by the column-free path");
        return s2_igrad_prepare(as_stream(stream), gy, w, scratch, g2, B, xch, ych, kh, kw, pad);
    }
    FusedGeom g;
    AG_REQUIRE(fused_geom(B, ych, yh, yw, xch, kh, kw, pad, xh, xw, &g, dilation) && aligned16(scratch), AG_ERR_INVALID_DIMS,
               "conv_input_grad_prepare: geometry not supported by the column-free path");
    return fused_prepare(as_stream(stream), gy, w, scratch, g, B, ych, yh, yw, xch, kh, kw, pad, dilation);
}

extern "C" ag_status_t ag_conv_input_grad_gemm_f32(ag_stream_t stream, float *scratch, float *gx, int B, int ych,
                                                   int yh, int yw, int xch, int kh, int kw, int pad, int stride, int dilation,
                                                   int xh, int xw)
{
    AG_REQUIRE(nocols_mode(stride, dilation), AG_ERR_INVALID_DIMS, "conv_input_grad_gemm: stride %d / dilation %d not supported",
               stride, dilation);
    AG_REQUIRE(scratch && gx, AG_ERR_INVALID_DIMS, "conv_input_grad_gemm: null pointer");
    if (stride == 2) {
        S2Geom g2;
        AG_REQUIRE(s2_geom(B, xch, xh, xw, ych, kh, kw, pad, &g2) && g2.OH == yh && g2.OW == yw && aligned16(scratch) && aligned16(gx),
                   AG_ERR_INVALID_DIMS, "conv_input_grad_gemm: geometry not supported by the column-free path");
        return s2_igrad_gemm(as_stream(stream), scratch, gx, g2, B, xch, ych, xh, xw);
    }
    FusedGeom g;
    AG_REQUIRE(fused_geom(B, ych, yh, yw, xch, kh, kw, pad, xh, xw, &g, dilation) && aligned16(scratch) && aligned16(gx),
               AG_ERR_INVALID_DIMS, "conv_input_grad_gemm: geometry not supported by the column-free path");
    return gemm_conv_input_grad(as_stream(stream), scratch + g.gyp_floats, scratch, gx, B, xch, ych, xh, xw, kh, kw, g.Hp,
                                g.Wp, dilation, g.ws_floats ? scratch + g.gyp_floats + g.wr_floats : nullptr, (size_t)g.ws_floats);
}
