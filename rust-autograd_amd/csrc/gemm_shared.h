// Declarations shared by the two GEMM translation units (register-staged kernel and host
// dispatch in gemm.hip, direct-to-LDS kernel in gemm_dl.hip).
#pragma once
#include "ag_internal.h"

namespace ag {

typedef float f32x16 __attribute__((ext_vector_type(16)));

enum { LK_VEC = 0, LK_SCALAR = 1, LMN = 2 };

struct GemmParams {
    const float *A;
    const float *B;
    float *C;
    int M, N, K;
    long long lda, ldb, ldc;
    long long sA, sB, sC;  // stride between independent batches
    long long sAk, sBk;    // stride between accumulated batches
    int kbatch;            // accumulated batches (>= 1)
    int kb_per_split;
    int splits;
    long long sCsplit;     // stride between the partial outputs of consecutive splits
    float alpha, beta;
    int tiles_m, tiles_n;
    unsigned total_blocks;
    // Folded batch (direct-to-LDS kernel only): A shared by all batches and B, C n-contiguous, so
    // the batches are laid side by side along n -- column g of the folded problem is column
    // g % n_img of batch g / n_img -- and N = batch * n_img is tiled without padding every batch.
    int n_img;  // 0 = not folded
    int n_off;  // folded: first column of this launch (a launch may cover a column range only)
    // Implicit input gradient of a stride-1 convolution (direct-to-LDS kernel, folded batch):
    // B is the zero-bordered upstream gradient [batch][K][Hp][conv_wp]; the accumulated "batches"
    // are the kh*kw filter taps, tap (ky, kx) reading B shifted by (kh-1-ky)*conv_wp + (kw-1-kx)
    // elements; column n of a batch is pixel (n / conv_wp, n % conv_wp), stored to the dense
    // [.., H, conv_w] output only when n % conv_wp < conv_w.  0 = ordinary GEMM.
    int conv_wp, conv_w, conv_kw;
    // Stride-2 input gradient, both column parities of row parity conv_pair_a in one product
    // (conv_pair_w != 0): row m of the result is (channel m / 2, column parity m % 2), column (i, j)
    // is pixel (2i + conv_pair_a, 2j + m % 2) of an output plane conv_pair_w wide, so the two parities
    // of a channel leave as one 8-byte store.  ldc / sC are the plane / image strides of that output.
    int conv_pair_w, conv_pair_a;
    // Pair form with its rows grouped by parity (conv_pair_grouped != 0): within every 64 rows of A the first 32 are
    // column parity 0 of 32 channels and the next 32 parity 1 of the same channels, so that one of a wave's two
    // 32-row MFMA blocks belongs to each parity; bit t of conv_pair_skip[b] says that parity b has no filter tap at
    // tap slot t of the union (its rows of A are zero there), and the kernel leaves those matrix instructions out.
    int conv_pair_grouped;
    unsigned conv_pair_skip[2];
    // Stride-2 forward (conv_phase != 0): B holds the four phase planes of the zero-bordered input,
    // [batch][K][2][2][Hpp][conv_wp] with phase (a, b) = elements (2i+a, 2j+b), conv_phase elements
    // each; tap (ky, kx), visited in natural order, reads phase (ky&1, kx&1) shifted by
    // (ky>>1)*conv_wp + (kx>>1) elements.
    unsigned conv_phase;
    // Implicit filter gradient of a stride-1 convolution (direct-to-LDS kernel, k-contiguous B): row n
    // of B is (channel n / rows_taps, tap n % rows_taps) of a zero-bordered input [..][C][Hp][rows_wp]
    // and starts (channel * rows_plane + ky * rows_wp + kx) elements after B; the contraction runs
    // over the flattened padded plane.  0 = rows of B are ldb apart.
    int rows_taps, rows_kw, rows_wp;
    unsigned rows_plane;
    unsigned rows_phase;  // != 0: stride-2 filter gradient, row (channel, ky, kx) starts at
                          // channel*rows_plane + ((ky&1)*2 + (kx&1))*rows_phase + (ky>>1)*rows_wp + (kx>>1)
    // Dilation of the stride-1 forms (input gradient and filter gradient): every tap shift above is multiplied by
    // it.  1 for the stride-2 forms.
    int conv_dil;
};

// Elements of the contraction that one accumulation chain of the MFMA kernels covers before its sum
// is set aside and the chain restarts from zero (both GEMM kernels).  OpenBLAS blocks its SGEMM
// contraction the same way; with 512 the error against an f64 result is 1.08 times OpenBLAS's at
// 4096^3 (256: 0.76 times, for twice the set-aside work; one chain of 4096: 6 times).
constexpr int kChainK = 512;

// Launches direct-to-LDS configuration `cfg` (kFirstDirectCfg ..); `ka` / `kb`: the operand is
// k-contiguous.  `blocks_per_cu` > 0 overrides the persistent grid size.
constexpr int kFirstDirectCfg = 13;
// `second`: see gemm_dl.hip (two grouped pair-form products in one launch).
void launch_direct(hipStream_t st, int cfg, bool ka, bool kb, const GemmParams &p, int cus, int blocks_per_cu,
                   const GemmParams *second = nullptr);
// Implicit filter gradient: gw[k][c][tap] = sum over images and positions q, counted from the first
// gradient value of a plane, of gyp[b][k][q + pad * Wp + pad] * xp[b][c][q + ky * Wp + kx].  gyp, xp:
// zero-bordered [B][.][Hp][Wp] with the same border `pad`; `kq` (a multiple of 32) positions cover
// every non-zero element of gyp and end inside the zero rows below it.  `ws`: partial sums of the
// split over images.
size_t gemm_conv_filter_grad_workspace(int B, int Kf, int C, int taps, int kq);
ag_status_t gemm_conv_filter_grad(hipStream_t st, const float *gyp, const float *xp, float *gw, void *ws, size_t ws_bytes,
                                  int B, int Kf, int C, int kh, int kw, int border, int Hp_gy, int Hp_x, int Wp, int kq,
                                  int dil = 1);
// `ws` / `ws_floats`: room for the partial results of a split contraction (gemm_conv_input_grad_ws_floats; may be
// null, then the contraction is not split).
ag_status_t gemm_conv_input_grad(hipStream_t st, const float *wr, const float *gyp, float *gx, int B, int C,
                                 int Kf, int H, int W, int kh, int kw, int Hp, int Wp, int dil = 1, float *ws = nullptr,
                                 size_t ws_floats = 0);
size_t gemm_conv_input_grad_ws_floats(int B, int C, int Kf, int H, int W, int Wp, int taps);
// Stride-2 forward over phase planes (see GemmParams::conv_phase): wf [K][kh*kw][C] in natural tap
// order, xph [B][C][4][Hpp][Wpp], y [B][K][OH][OW].
// The pair form of the implicit input gradient (see GemmParams::conv_pair_w): wr [2C][kh*kw*Kf], gyp bordered
// upstream gradient, gx [B][C][Hout][Wout] receives rows 2i + a, i < Ha, and columns 2j + b, j < Wb.
// `skip` != null: the rows of wr are grouped by parity and skip[b] lists the tap slots at which parity b is zero
// (GemmParams::conv_pair_grouped); gemm_conv_input_grad_pair_grouped says whether the product of these extents
// runs on a tile that supports it (the filter must be written accordingly).
ag_status_t gemm_conv_input_grad_pair(hipStream_t st, const float *wr, const float *gyp, float *gx, int B, int C, int Kf, int Ha,
                                      int Wb, int kh, int kw, int Hp, int Wp, int a, int Hout, int Wout,
                                      const unsigned *skip = nullptr);
bool gemm_conv_input_grad_pair_grouped(int B, int C, int Kf, int Ha, int Wp, int taps);
// Both row parities of the grouped pair form (skip[a] non-null for both), merged into shared launches where their tiles
// agree; arguments indexed by the row parity a are those of two gemm_conv_input_grad_pair calls.
ag_status_t gemm_conv_input_grad_pair_both(hipStream_t st, const float *const wr[2], const float *const gyp[2], float *gx, int B,
                                           int C, int Kf, const int Ha[2], int Wb, const int kh[2], int kw, int Hp, int Wp,
                                           int Hout, int Wout, const unsigned *const skip[2]);
ag_status_t gemm_conv_fwd_stride2(hipStream_t st, const float *wf, const float *xph, float *y, int B, int K, int C,
                                  int OH, int OW, int kh, int kw, int Hpp, int Wpp);
// Stride-2 filter gradient: gw[k][c][ky][kx] = sum over images and positions q of
// gyq[b][k][q] * xph[b][c][phase(ky,kx)][q + (ky>>1)*Wpp + (kx>>1)]; gyq [B][K][Hq][Wpp] holds gy at row
// pitch Wpp with zeros elsewhere; kq (a multiple of 32) positions.
size_t gemm_conv_filter_grad_stride2_workspace(int B, int Kf, int C, int taps);
ag_status_t gemm_conv_filter_grad_stride2(hipStream_t st, const float *gyq, const float *xph, float *gw, void *ws,
                                          size_t ws_bytes, int B, int Kf, int C, int kh, int kw, int Hq, int Hpp, int Wpp, int kq);
// Direct-to-LDS configuration with a 64-row tile (64 x 128, two blocks per CU), used by the implicit input gradient.
constexpr int kDirectCfg64 = 19;
constexpr int kDirectCfg32 = 20;        // 32 x 128, k-contiguous A only
constexpr int kDirectCfg64Narrow = 21;  // 64 x 64

}  // namespace ag
