// Column-free stride-2 convolution: forward, filter gradient and input gradient as implicit GEMMs.
// No counterpart in the reference, which materialises the im2col columns for every stride
// (conv2d.rs:25-112, 631-734; conv2d_transpose.rs:89-247); the index arithmetic restated here is
// that of conv_ops/mod.rs:89-112 (x index = o*stride - pad + k) and its adjoint (:198-219).
//
// A stride-2 window reads x'[2*oy + ky][2*ox + kx] (x' = x with a zero border of `pad`).  Splitting
// x' into its four PHASE planes x'_{a,b}[i][j] = x'[2i+a][2j+b] turns that into the unit-stride read
// x'_{ky&1,kx&1}[oy + (ky>>1)][ox + (kx>>1)], so
//   forward          y  = sum over taps and channels of w * phase plane shifted by (ky>>1, kx>>1)  -- one GEMM;
//   filter gradient  gw[k][c][ky][kx] = sum over images and positions q of gy'[k][q] * x'_{..}[c][q + shift]  -- one GEMM;
//   input gradient   the pixels of one parity (iy&1, ix&1) of gx only meet the taps with ky = iy + pad and
//                    kx = ix + pad (mod 2): four unit-stride input-gradient GEMMs, one per parity, over ONE
//                    zero-bordered copy of gy; their results (parity-planar) are interleaved into gx by a copy kernel.
// All planes share one row pitch Wc, so the bordered gy serves the filter gradient as well.
#include "ag_internal.h"
#include "conv_shared.h"
#include "gemm_shared.h"

namespace ag {

static long long round_up32(long long v) { return (v + 31) / 32 * 32; }

bool s2_geom(int B, int C, int H, int W, int K, int kh, int kw, int pad, S2Geom *g)
{
    if (B < 1 || C < 1 || K < 1 || H < 1 || W < 1 || kh < 2 || kw < 2 || pad < 0 || pad > kh - 1 || pad > kw - 1) return false;
    if (C % 32 != 0 || K % 32 != 0) return false;
    if (H + 2 * pad < kh || W + 2 * pad < kw) return false;
    g->OH = (H + 2 * pad - kh) / 2 + 1;
    g->OW = (W + 2 * pad - kw) / 2 + 1;
    // parities of the input gradient: which taps they meet and how far they reach into gy
    int T = 0, L = 0, reach_h = 0, reach_w = 0;
    for (int a = 0; a < 2; ++a) {
        const int alpha = (a + pad) & 1;
        g->kh_a[a] = (kh - alpha + 1) / 2;
        g->kw_b[a] = (kw - alpha + 1) / 2;
        g->d_a[a] = (a + pad) >> 1;
        g->H_a[a] = (H - a + 1) / 2;
        g->W_b[a] = (W - a + 1) / 2;
        T = T > g->kh_a[a] - 1 - g->d_a[a] ? T : g->kh_a[a] - 1 - g->d_a[a];
        L = L > g->kw_b[a] - 1 - g->d_a[a] ? L : g->kw_b[a] - 1 - g->d_a[a];
        L = L > g->d_a[a] ? L : g->d_a[a];  // a read past the end of a row lands in the next row's left border
        reach_h = reach_h > g->H_a[a] + g->d_a[a] ? reach_h : g->H_a[a] + g->d_a[a];
        reach_w = reach_w > g->W_b[a] + g->d_a[a] ? reach_w : g->W_b[a] + g->d_a[a];
    }
    g->T = T;
    g->L = L;
    // common row pitch: wide enough for the phase planes and for the bordered gy; every per-image column
    // range that a GEMM folds along n (OH*Wc forward, H_a*Wc input gradient) a multiple of four elements
    int Wc = g->OW + (kw - 1) / 2;
    if (Wc < L + g->OW) Wc = L + g->OW;
    if (Wc < reach_w) Wc = reach_w;
    const int first = Wc;
    for (;; ++Wc) {
        if (Wc > first + 8) return false;
        if (((long long)g->OH * Wc) % 4 == 0 && ((long long)g->H_a[0] * Wc) % 4 == 0 &&
            (g->H_a[1] == 0 || ((long long)g->H_a[1] * Wc) % 4 == 0))
            break;
    }
    g->Wc = Wc;
    g->kq = (int)round_up32((long long)g->OH * Wc);
    // phase planes of x': every tap of every output lies inside, and so does everything the filter
    // gradient reads while its positions run up to kq (against zeros of gy')
    g->Hpp = g->OH + (kh - 1) / 2;
    while (((long long)g->Hpp * Wc) % 4 != 0 || (long long)g->Hpp * Wc < g->kq + (long long)((kh - 1) / 2) * Wc + (kw - 1) / 2) ++g->Hpp;
    g->pp = (long long)g->Hpp * Wc;
    // bordered gy: rows for the deepest reach of the input gradient and for the kq positions of the filter gradient
    g->Hp = T + (g->OH > reach_h ? g->OH : reach_h);
    while (((long long)g->Hp * Wc) % 4 != 0 || (long long)g->Hp * Wc < (long long)T * Wc + L + g->kq) ++g->Hp;
    g->xph_floats = (long long)B * C * 4 * g->pp + kS2Slack;
    g->wf_floats = (long long)K * C * kh * kw;
    g->gyp_floats = (long long)B * K * g->Hp * Wc + kS2Slack;
    g->gxp_floats = (long long)B * C * H * W;
    if (g->pp / 4 >= 32768) return false;  // range of the multiply-high divisions of the phase split
    // 128-column tiles may straddle two images, not three; 32-bit offsets inside one image
    if ((long long)g->OH * Wc < 128 || (long long)g->H_a[0] * Wc < 128 || (g->H_a[1] > 0 && (long long)g->H_a[1] * Wc < 128)) return false;
    if ((long long)B * g->Hpp * Wc >= 0x7fffffffLL || (long long)C * 4 * g->pp >= (1LL << 30) ||
        (long long)K * g->Hp * Wc >= (1LL << 30))
        return false;
    return true;
}

// xph[b][c][a][b'][i][j] = x'[2i+a][2j+b'] = x[b][c][2i+a-pad][2j+b'-pad], zero outside x; grid.y walks the
// (image, channel) planes.  One thread per four consecutive elements of BOTH column phases of a row phase a: the
// eight inputs x[2i+a-pad][2j-pad .. 2j+7-pad] are neighbours in memory (two 16-byte loads that need only
// 4-byte alignment when the quad lies inside one row and inside the image), the even ones go to phase (a,0) and
// the odd ones to phase (a,1).  A wave then uses every byte of the cache lines it touches; with a thread per
// phase each line was fetched twice, by threads far apart in the grid.
struct __attribute__((packed, aligned(4))) F4U {
    float x, y, z, w;
};

// The last `extra_rows` rows of the grid split nothing: they zero the slack after the planes and write the filter as the
// k-contiguous left operand of the forward GEMM, wf[k][tap][c] = w[k][c][tap], so that the preparation is one launch.
__global__ __launch_bounds__(256) void phase_split_pair_kernel(const float *__restrict__ x, float *__restrict__ xph, int planes,
                                                               int H, int W, int pad, int Wc, unsigned quads_phase,
                                                               unsigned m_phase, unsigned m_row, float *__restrict__ slack,
                                                               int n_slack, const float *__restrict__ w,
                                                               float *__restrict__ wf, int K, int C, int taps,
                                                               unsigned extra_rows)
{
    const unsigned ny = gridDim.y - extra_rows;
    if (blockIdx.y >= ny) {
        const int tid = (int)(((blockIdx.y - ny) * gridDim.x + blockIdx.x) * 256u + threadIdx.x);
        const int nth = (int)(extra_rows * gridDim.x * 256u);
        for (int e = tid; e < n_slack; e += nth) slack[e] = 0.f;
        const int total = K * C * taps;
        for (int e = tid; e < total; e += nth) {
            const int c = e % C, tap = e / C % taps, k = e / (C * taps);
            wf[e] = w[((long long)k * C + c) * taps + tap];
        }
        return;
    }
    const unsigned qi = blockIdx.x * 256u + threadIdx.x;  // quad inside the two row phases of one channel
    if (qi >= 2u * quads_phase) return;
    const unsigned a = __umulhi(qi, m_phase);
    const unsigned q = qi - a * quads_phase;
    const unsigned e0 = q * 4u;
    int i = (int)__umulhi(e0, m_row), j = (int)(e0 - (unsigned)i * (unsigned)Wc);
    const int r0 = 2 * i + (int)a - pad, s0 = 2 * j - pad;
    const bool fast = j + 3 < Wc && (unsigned)r0 < (unsigned)H && s0 >= 0 && s0 + 7 < W;
    int off[8];
    bool in[8];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int r = 2 * i + (int)a - pad;
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const int sx = 2 * j + b - pad;
            in[2 * t + b] = (unsigned)r < (unsigned)H && (unsigned)sx < (unsigned)W;
            off[2 * t + b] = r * W + sx;
        }
        if (++j == Wc) {
            j = 0;
            ++i;
        }
    }
    const long long phase_pair = 2LL * quads_phase;  // float4 units of the two column phases of one row phase
    for (int pl = blockIdx.y; pl < planes; pl += ny) {
        const float *src = x + (long long)pl * H * W;
        float v[8];
        if (fast) {
            const F4U lo = *reinterpret_cast<const F4U *>(src + off[0]);
            const F4U hi = *reinterpret_cast<const F4U *>(src + off[0] + 4);
            v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w;
            v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
        } else {
#pragma unroll
            for (int t = 0; t < 8; ++t) v[t] = in[t] ? src[off[t]] : 0.f;
        }
        float4 *dst = reinterpret_cast<float4 *>(xph) + ((long long)pl * 2 + a) * phase_pair + q;
        st_stream(dst, make_float4(v[0], v[2], v[4], v[6]));
        st_stream(dst + quads_phase, make_float4(v[1], v[3], v[5], v[7]));
    }
}

__global__ void s2_zero_kernel(float *p, int n)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) p[i] = 0.f;
}

// wf[k][tap][c] = w[k][c][tap]: the filter as the k-contiguous left operand of the stride-2 forward GEMM.
__global__ __launch_bounds__(256) void s2_filter_fwd_kernel(const float *__restrict__ w, float *__restrict__ wf, int K, int C,
                                                            int taps)
{
    const int total = K * C * taps;
    for (int e = blockIdx.x * 256 + threadIdx.x; e < total; e += gridDim.x * 256) {
        const int c = e % C, tap = e / C % taps, k = e / (C * taps);
        wf[e] = w[((long long)k * C + c) * taps + tap];
    }
}

// The four sub-filters of the input gradient, one per output parity (a, b), back to back:
// wr_ab[c][m*kw_b + n][k] = w[k][c][2m + alpha_a][2n + alpha_b]  (k fastest).
__global__ __launch_bounds__(256) void s2_filter_parity_kernel(const float *__restrict__ w, float *__restrict__ wr, int K, int C,
                                                               int kh, int kw, int pad)
{
    const int total = K * C * kh * kw;
    for (int e = blockIdx.x * 256 + threadIdx.x; e < total; e += gridDim.x * 256) {
        // destination element e: find its parity block
        int rest = e, a = 0, b = 0, kha = 0, kwb = 0;
        for (int ph = 0; ph < 4; ++ph) {
            a = ph >> 1;
            b = ph & 1;
            kha = (kh - ((a + pad) & 1) + 1) / 2;
            kwb = (kw - ((b + pad) & 1) + 1) / 2;
            const int size = C * kha * kwb * K;
            if (rest < size) break;
            rest -= size;
        }
        const int k = rest % K, tap = rest / K % (kha * kwb), c = rest / (K * kha * kwb);
        const int m = tap / kwb, n = tap - m * kwb;
        const int ky = 2 * m + ((a + pad) & 1), kx = 2 * n + ((b + pad) & 1);
        wr[e] = w[(((long long)k * C + c) * kh + ky) * kw + kx];
    }
}

// The pair form of the input gradient (even W): for a row parity a, the two column parities b of a channel are
// rows 2c + b of ONE product whose taps are the union of the two parities' column shifts (parity b reads gy shifted
// by d_b - n columns for its tap n; the union is smin .. smax, visited from smax down), with zeros where a parity
// has no tap at a shift.  The GEMM's epilogue then writes gx[c][2i+a][2j .. 2j+1] as one 8-byte store, so no
// parity-planar intermediate and no interleaving pass exist; the price is the zero taps (3 x 3, pad 1: 12 instead of
// 9 tap-products per channel pair) on tiles of 128 rows instead of 64.
// Where the product of a row parity runs on a tile whose waves hold 64 rows, the rows are grouped by parity instead
// (of every 64 rows the first 32 are column parity 0 of 32 channels, the next 32 parity 1 of the same channels): one
// of a wave's two 32-row blocks then belongs to each parity, and the kernel leaves out the matrix instructions of a
// parity at the shifts where it has no tap -- the zero taps cost loads of zeros but no matrix time (3 x 3, pad 1: the
// work of 9 tap-products per channel pair again; 4 x 4, pad 1: 8 instead of 12).
struct S2Pair {
    int smax, kwp;           // largest column shift, number of shifts in the union
    long long floats[2];     // elements of the merged filter of row parity a
    int grouped[2];          // rows of row parity a's filter grouped by column parity
    unsigned skip[2][2];     // [a][b]: tap slots (m * kwp + n') of row parity a at which column parity b has no tap
};

static bool s2_pair(const S2Geom &g, int B, int C, int K, int W, S2Pair *pr)
{
    if (W % 2 != 0 || g.W_b[0] != g.W_b[1] || g.W_b[0] < 1 || g.kw_b[0] < 1 || g.kw_b[1] < 1) return false;
    const int smax = g.d_a[0] > g.d_a[1] ? g.d_a[0] : g.d_a[1];
    const int lo0 = g.d_a[0] - g.kw_b[0] + 1, lo1 = g.d_a[1] - g.kw_b[1] + 1;
    const int smin = lo0 < lo1 ? lo0 : lo1;
    if (g.L + smin < 0) return false;
    pr->smax = smax;
    pr->kwp = smax - smin + 1;
    for (int a = 0; a < 2; ++a) {
        pr->floats[a] = 2LL * C * g.kh_a[a] * pr->kwp * K;
        const int slots = g.kh_a[a] * pr->kwp;
        pr->grouped[a] = g.H_a[a] > 0 && slots <= 32 && gemm_conv_input_grad_pair_grouped(B, C, K, g.H_a[a], g.Wc, slots);
        for (int b = 0; b < 2; ++b) {
            pr->skip[a][b] = 0;
            for (int t = 0; t < slots && t < 32; ++t) {
                const int n = t % pr->kwp - (smax - g.d_a[b]);
                if (n < 0 || n >= g.kw_b[b]) pr->skip[a][b] |= 1u << t;
            }
        }
    }
    // the merged filters take the place of the parity filters and of the parity-planar result
    return pr->floats[0] + pr->floats[1] <= g.wf_floats + g.gxp_floats && pr->floats[0] + pr->floats[1] < 0x7fffffffLL;
}

// wp_a[2c + b][m * kwp + n'][k] = w[k][c][2m + alpha_a][2n + alpha_b] with n = n' - (smax - d_b), or 0 when parity b
// has no tap n there; the filters of a = 0 and a = 1 back to back.
// `grouped0` / `grouped1`: the rows of that row parity's filter are grouped by column parity (row = 64 * (c / 32) +
// 32 * b + c % 32) instead of interleaved (row = 2c + b).
__global__ __launch_bounds__(256) void s2_filter_pair_kernel(const float *__restrict__ w, float *__restrict__ wp, int K, int C,
                                                             int kh, int kw, int pad, int smax, int kwp, int size0, int total,
                                                             int grouped0, int grouped1, float *__restrict__ slack, int n_slack)
{
    // (also zeroes the slack behind the bordered gradient, so that the preparation needs no launch for that)
    for (int e = blockIdx.x * 256 + threadIdx.x; e < n_slack; e += gridDim.x * 256) slack[e] = 0.f;
    for (int e = blockIdx.x * 256 + threadIdx.x; e < total; e += gridDim.x * 256) {
        const int a = e >= size0, rest = a ? e - size0 : e;
        const int alpha_a = (a + pad) & 1, kha = (kh - alpha_a + 1) / 2;
        const int k = rest % K, tap = rest / K % (kha * kwp), row = rest / (K * kha * kwp);
        const bool grouped = a ? grouped1 != 0 : grouped0 != 0;
        const int c = grouped ? (row >> 6) * 32 + (row & 31) : row >> 1, b = grouped ? (row >> 5) & 1 : row & 1;
        const int alpha_b = (b + pad) & 1, kwb = (kw - alpha_b + 1) / 2, d_b = (b + pad) >> 1;
        const int m = tap / kwp, n = tap - m * kwp - (smax - d_b);
        float v = 0.f;
        if (n >= 0 && n < kwb) v = w[(((long long)k * C + c) * kh + 2 * m + alpha_a) * kw + 2 * n + alpha_b];
        wp[e] = v;
    }
}

// gx[pl][2i+a][2j+b] = gxp_ab[pl][i][j]: four consecutive pixels of a row per thread (W % 4 == 0), or one.
__global__ __launch_bounds__(256) void s2_interleave_kernel(const float *__restrict__ gxp, float *__restrict__ gx, long long planes,
                                                            int H, int W, int H0, int H1, int W0, int W1, int vec)
{
    const long long o00 = 0, o01 = planes * H0 * W0, o10 = o01 + planes * H0 * W1, o11 = o10 + planes * H1 * W0;
    if (vec) {
        const long long quads = planes * H * (W / 4);
        for (long long q = blockIdx.x * 256LL + threadIdx.x; q < quads; q += gridDim.x * 256LL) {
            const int xq = (int)(q % (W / 4));
            const long long t = q / (W / 4);
            const int iy = (int)(t % H);
            const long long pl = t / H;
            const int i = iy >> 1, j = 2 * xq;
            const float *e, *o;  // even and odd columns of this row
            if (iy & 1) {
                e = gxp + o10 + (pl * H1 + i) * W0 + j;
                o = gxp + o11 + (pl * H1 + i) * W1 + j;
            } else {
                e = gxp + o00 + (pl * H0 + i) * W0 + j;
                o = gxp + o01 + (pl * H0 + i) * W1 + j;
            }
            st_stream(reinterpret_cast<float4 *>(gx) + q, make_float4(e[0], o[0], e[1], o[1]));
        }
    } else {
        const long long total = planes * H * W;
        for (long long q = blockIdx.x * 256LL + threadIdx.x; q < total; q += gridDim.x * 256LL) {
            const int ix = (int)(q % W);
            const long long t = q / W;
            const int iy = (int)(t % H);
            const long long pl = t / H;
            const int i = iy >> 1, j = ix >> 1;
            const int Ha = (iy & 1) ? H1 : H0, Wb = (ix & 1) ? W1 : W0;
            const long long base = (iy & 1) ? ((ix & 1) ? o11 : o10) : ((ix & 1) ? o01 : o00);
            gx[q] = gxp[base + (pl * Ha + i) * Wb + j];
        }
    }
}

static unsigned magic(unsigned d) { return (unsigned)((1ULL << 32) / d) + 1u; }

ag_status_t s2_fwd_prepare(hipStream_t st, const float *x, const float *w, float *xpad, const S2Geom &g, int B, int C, int H,
                           int W, int K, int kh, int kw, int pad)
{
    const unsigned quads_phase = (unsigned)(g.pp / 4);
    const long long planes = (long long)B * C;
    // one grid row per (image, channel) plane, plus enough rows for a thread per filter element (256 blocks at most)
    const unsigned gx_blocks = (2 * quads_phase + 255) / 256;
    unsigned extra_rows = (unsigned)((g.wf_floats + 255) / 256 + gx_blocks - 1) / gx_blocks;
    if (extra_rows * gx_blocks > 256) extra_rows = (256 + gx_blocks - 1) / gx_blocks;
    if (extra_rows < 1) extra_rows = 1;
    const dim3 grid(gx_blocks, (unsigned)(planes < 65535 - extra_rows ? planes : 65535 - extra_rows) + extra_rows);
    hipLaunchKernelGGL(phase_split_pair_kernel, grid, dim3(256), 0, st, x, xpad, (int)planes, H, W, pad, g.Wc, quads_phase,
                       magic(quads_phase), magic((unsigned)g.Wc), xpad + planes * 4 * g.pp, (int)kS2Slack, w,
                       xpad + g.xph_floats, K, C, kh * kw, extra_rows);
    return check_launch("conv2d");
}

ag_status_t s2_fwd_filter(hipStream_t st, const float *w, float *wf, const S2Geom &g, int C, int K, int kh, int kw)
{
    hipLaunchKernelGGL(s2_filter_fwd_kernel, dim3((unsigned)((g.wf_floats + 255) / 256)), dim3(256), 0, st, w, wf, K, C, kh * kw);
    return check_launch("conv2d");
}

ag_status_t s2_fwd_gemm(hipStream_t st, const float *xph, const float *wf, float *y, const S2Geom &g, int B, int C, int K, int kh,
                        int kw)
{
    return gemm_conv_fwd_stride2(st, wf, xph, y, B, K, C, g.OH, g.OW, kh, kw, g.Hpp, g.Wc);
}

// Scratch of the input gradient: zero-bordered gy, the four parity filters, the parity-planar result.
ag_status_t s2_igrad_prepare(hipStream_t st, const float *gy, const float *w, float *scratch, const S2Geom &g, int B, int C, int K,
                             int kh, int kw, int pad)
{
    launch_pad_border(st, gy, scratch, B, K, g.OH, g.OW, g.Hp, g.Wc, g.T, g.L);
    float *slack = scratch + (long long)B * K * g.Hp * g.Wc;
    S2Pair pr;
    if (s2_pair(g, B, C, K, g.W_b[0] + g.W_b[1], &pr)) {
        const int total = (int)(pr.floats[0] + pr.floats[1]);
        hipLaunchKernelGGL(s2_filter_pair_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, w, scratch + g.gyp_floats,
                           K, C, kh, kw, pad, pr.smax, pr.kwp, (int)pr.floats[0], total, pr.grouped[0], pr.grouped[1], slack,
                           (int)kS2Slack);
    } else {
        hipLaunchKernelGGL(s2_zero_kernel, dim3(4), dim3(256), 0, st, slack, (int)kS2Slack);
        hipLaunchKernelGGL(s2_filter_parity_kernel, dim3((unsigned)((g.wf_floats + 255) / 256)), dim3(256), 0, st, w,
                           scratch + g.gyp_floats, K, C, kh, kw, pad);
    }
    return check_launch("conv2d_transpose");
}

ag_status_t s2_igrad_gemm(hipStream_t st, float *scratch, float *gx, const S2Geom &g, int B, int C, int K, int H, int W)
{
    const float *gyp = scratch;
    const float *wr = scratch + g.gyp_floats;
    S2Pair pr;
    if (s2_pair(g, B, C, K, W, &pr)) {
        // (the prepare step has written the merged filters, so there is no falling back to the parity form here)
        AG_REQUIRE((reinterpret_cast<uintptr_t>(gx) & 7) == 0, AG_ERR_INVALID_DIMS,
                   "conv2d_transpose (column-free, stride 2): the output must be 8-byte aligned");
        if (g.H_a[0] > 0 && g.H_a[1] > 0 && pr.grouped[0] && pr.grouped[1]) {
            const float *wrs[2] = {wr, wr + pr.floats[0]}, *origins[2];
            const unsigned *skips[2] = {pr.skip[0], pr.skip[1]};
            for (int a = 0; a < 2; ++a)
                origins[a] = gyp + (long long)(g.T - (g.kh_a[a] - 1 - g.d_a[a])) * g.Wc + (g.L + pr.smax - (pr.kwp - 1));
            return gemm_conv_input_grad_pair_both(st, wrs, origins, gx, B, C, K, g.H_a, g.W_b[0], g.kh_a, pr.kwp, g.Hp, g.Wc, H, W,
                                                  skips);
        }
        for (int a = 0; a < 2; ++a) {
            if (g.H_a[a] > 0) {
                const int top = g.kh_a[a] - 1 - g.d_a[a];
                // the first shift the GEMM visits is the largest: origin + (kwp - 1) = L + smax
                const float *origin = gyp + (long long)(g.T - top) * g.Wc + (g.L + pr.smax - (pr.kwp - 1));
                if (ag_status_t s = gemm_conv_input_grad_pair(st, wr, origin, gx, B, C, K, g.H_a[a], g.W_b[0], g.kh_a[a], pr.kwp,
                                                              g.Hp, g.Wc, a, H, W, pr.grouped[a] ? pr.skip[a] : nullptr))
                    return s;
            }
            wr += pr.floats[a];
        }
        return AG_OK;
    }
    float *gxp = scratch + g.gyp_floats + g.wf_floats;
    long long out_off = 0;
    for (int a = 0; a < 2; ++a)
        for (int b = 0; b < 2; ++b) {
            const int kha = g.kh_a[a], kwb = g.kw_b[b], Ha = g.H_a[a], Wb = g.W_b[b];
            const long long wsize = (long long)C * kha * kwb * K;
            if (Ha > 0 && Wb > 0) {
                // this parity's own borders inside the shared copy
                const int top = kha - 1 - g.d_a[a], left = kwb - 1 - g.d_a[b];
                const float *origin = gyp + (long long)(g.T - top) * g.Wc + (g.L - left);
                if (ag_status_t s = gemm_conv_input_grad(st, wr, origin, gxp + out_off, B, C, K, Ha, Wb, kha, kwb, g.Hp, g.Wc))
                    return s;
            }
            wr += wsize;
            out_off += (long long)B * C * Ha * Wb;
        }
    const long long planes = (long long)B * C;
    const int vec = (W % 4 == 0) && aligned16(gx);
    long long blocks = ((vec ? planes * H * (W / 4) : planes * H * W) + 255) / 256;
    if (blocks > 1048576) blocks = 1048576;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(s2_interleave_kernel, dim3((unsigned)blocks), dim3(256), 0, st, gxp, gx, planes, H, W, g.H_a[0], g.H_a[1],
                       g.W_b[0], g.W_b[1], vec);
    return check_launch("conv2d_transpose");
}

size_t s2_filter_grad_workspace(const S2Geom &, int B, int C, int K, int kh, int kw)
{
    return gemm_conv_filter_grad_stride2_workspace(B, K, C, kh * kw);
}

ag_status_t s2_filter_grad(hipStream_t st, const float *xph, const float *gyp, float *gw, const S2Geom &g, int B, int C, int K,
                           int kh, int kw, void *ws, size_t ws_bytes)
{
    // positions are counted from the first gradient value of a bordered plane
    return gemm_conv_filter_grad_stride2(st, gyp + ((long long)g.T * g.Wc + g.L), xph, gw, ws, ws_bytes, B, K, C, kh, kw, g.Hp,
                                         g.Hpp, g.Wc, g.kq);
}

}  // namespace ag
