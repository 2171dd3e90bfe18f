// Declarations shared by the convolution translation units (conv.hip: operators and the
// unit-stride column-free path; conv_s2.hip: the stride-2 column-free path).
#pragma once
#include "ag_internal.h"

namespace ag {

// Zero-bordered copy of `planes` planes per image: dst[b][pl][r][s] = src[b][pl][r - top][s - left]
// inside the image, 0 elsewhere; dst planes are Hp x Wp with Hp * Wp a multiple of four.
void launch_pad_border(hipStream_t st, const float *src, float *dst, int B, int planes, int OH, int OW, int Hp, int Wp,
                       int top, int left);

constexpr long long kS2Slack = 1024;  // zeroed floats after the planes of a stride-2 scratch buffer

// Geometry of the column-free stride-2 convolution x [B,C,H,W] * w [K,C,kh,kw] -> y [B,K,OH,OW].
struct S2Geom {
    int OH, OW;
    int Wc;        // row pitch shared by the phase planes of x' and the bordered gy
    int Hpp;       // rows of a phase plane
    long long pp;  // Hpp * Wc
    int T, L, Hp;  // bordered gy: top and left border, rows
    int kq;        // positions the filter gradient contracts over (a multiple of 32)
    // per parity (index a for rows, b for columns) of the input gradient: taps, reach into gy, extent
    int kh_a[2], kw_b[2], d_a[2], H_a[2], W_b[2];
    long long xph_floats, wf_floats, gyp_floats, gxp_floats;
};
bool s2_geom(int B, int C, int H, int W, int K, int kh, int kw, int pad, S2Geom *g);
ag_status_t s2_fwd_prepare(hipStream_t st, const float *x, const float *w, float *xpad, const S2Geom &g, int B, int C, int H,
                           int W, int K, int kh, int kw, int pad);
ag_status_t s2_fwd_filter(hipStream_t st, const float *w, float *wf, const S2Geom &g, int C, int K, int kh, int kw);
ag_status_t s2_fwd_gemm(hipStream_t st, const float *xph, const float *wf, float *y, const S2Geom &g, int B, int C, int K, int kh,
                        int kw);
ag_status_t s2_igrad_prepare(hipStream_t st, const float *gy, const float *w, float *scratch, const S2Geom &g, int B, int C, int K,
                             int kh, int kw, int pad);
ag_status_t s2_igrad_gemm(hipStream_t st, float *scratch, float *gx, const S2Geom &g, int B, int C, int K, int H, int W);
size_t s2_filter_grad_workspace(const S2Geom &g, int B, int C, int K, int kh, int kw);
ag_status_t s2_filter_grad(hipStream_t st, const float *xph, const float *gyp, float *gw, const S2Geom &g, int B, int C, int K,
                           int kh, int kw, void *ws, size_t ws_bytes);

}  // namespace ag
