// fp32 GEMM on the CDNA matrix cores (v_mfma_f32_32x32x2_f32), the dense contraction under
// Conv2D forward, Conv2DFilterGrad, Conv2DTranspose, MatMul and BatchMatMul.
//
// One kernel family, templated on the block tile (BM x BN x BK), the per-wave tile (WM x WN) and
// how each operand is laid out in memory:
//   LK_VEC / LK_SCALAR  the reduction index k is the contiguous one (A not transposed, or B
//                       transposed): rows are fetched with 128-bit (or, when unaligned, 32-bit)
//                       loads along k;
//   LMN                 the m (or n) index is contiguous (A transposed, or B not transposed):
//                       lanes walk along m/n so every 32-bit load is coalesced across the wave
//                       and four k values are gathered per lane.
// Either way a tile lands in LDS as [row][k] with k contiguous and a 4-float pad per row, so each
// lane feeds four consecutive MFMA steps from one conflict-free 128-bit LDS read: in step s
// lanes 0-31 supply k = 8*kk+s and lanes 32-63 supply k = 8*kk+4+s, identically for A and B (the
// order in which k is consumed is free as long as both operands agree).
//
// Global loads for tile t+1 are issued into registers before the MFMA work of tile t and written
// to the other LDS buffer afterwards, so one barrier per tile suffices.
//
// A launch covers tiles x independent batches x splits; a "split" owns a contiguous range of the
// accumulated batch (the image-sequential beta=1 loop of the reference's filter gradients) and
// writes a partial result that a second fixed-order kernel folds, keeping the result
// deterministic.  Block ids are permuted so that each XCD (which has its own L2) works on a
// contiguous range of tiles / images.
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
};

constexpr int kXcds = 8;

// Hardware hands consecutive workgroup ids to the XCDs round-robin; give XCD x the x-th
// contiguous slice of the logical block range instead.
__device__ inline unsigned xcd_remap(unsigned id, unsigned total)
{
    const unsigned per = total / kXcds, rem = total % kXcds;
    const unsigned xcd = id % kXcds, pos = id / kXcds;
    return xcd * per + (xcd < rem ? xcd : rem) + pos;
}

template <int LT, int ROWS, int BK, int NT>
struct TileLoader {
    static constexpr int QUADS = BK / 4;
    static constexpr int PASSES = ROWS * BK / (4 * NT);
    static_assert(ROWS * BK % (4 * NT) == 0 && PASSES >= 1, "tile does not divide over the block");
    // k-contiguous mapping
    static constexpr int RPP = NT / QUADS;  // rows per pass
    // mn-contiguous mapping
    static constexpr int GROUPS = NT / ROWS > 0 ? NT / ROWS : 1;
    static_assert(LT != LMN || (NT % ROWS == 0 && QUADS % GROUPS == 0), "mn-contiguous mapping needs NT % ROWS == 0");
    static_assert(LT == LMN || (NT % QUADS == 0 && ROWS % RPP == 0), "k-contiguous mapping needs ROWS % (NT/(BK/4)) == 0");

    // Fetch this thread's share of the tile whose first row is row0 and first k is k0.
    // `base` already points at the right batch.  Out-of-range rows and k read as zero.
    __device__ static inline void load(const float *__restrict__ base, long long ld, int row0, int rows,
                                       int k0, int K, int tid, float4 (&r)[PASSES])
    {
        if (LT == LMN) {
            const int idx = tid % ROWS, grp = tid / ROWS;
            const bool row_ok = row0 + idx < rows;
            const float *p = base + row0 + idx;
#pragma unroll
            for (int ps = 0; ps < PASSES; ++ps) {
                const int k = k0 + (ps * GROUPS + grp) * 4;
                float4 v;
                v.x = (row_ok && k + 0 < K) ? p[(long long)(k + 0) * ld] : 0.f;
                v.y = (row_ok && k + 1 < K) ? p[(long long)(k + 1) * ld] : 0.f;
                v.z = (row_ok && k + 2 < K) ? p[(long long)(k + 2) * ld] : 0.f;
                v.w = (row_ok && k + 3 < K) ? p[(long long)(k + 3) * ld] : 0.f;
                r[ps] = v;
            }
        } else {
            const int rr = tid / QUADS, kq = (tid % QUADS) * 4;
            const int k = k0 + kq;
#pragma unroll
            for (int ps = 0; ps < PASSES; ++ps) {
                const int row = row0 + ps * RPP + rr;
                const float *p = base + (long long)row * ld + k;
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (row < rows) {
                    if (LT == LK_VEC) {
                        if (k < K) v = *reinterpret_cast<const float4 *>(p);  // K % 4 == 0 here
                    } else {
                        if (k + 0 < K) v.x = p[0];
                        if (k + 1 < K) v.y = p[1];
                        if (k + 2 < K) v.z = p[2];
                        if (k + 3 < K) v.w = p[3];
                    }
                }
                r[ps] = v;
            }
        }
    }

    __device__ static inline void store(float *__restrict__ lds, int ldk, int tid, const float4 (&r)[PASSES])
    {
        if (LT == LMN) {
            const int idx = tid % ROWS, grp = tid / ROWS;
#pragma unroll
            for (int ps = 0; ps < PASSES; ++ps)
                *reinterpret_cast<float4 *>(lds + idx * ldk + (ps * GROUPS + grp) * 4) = r[ps];
        } else {
            const int rr = tid / QUADS, kq = (tid % QUADS) * 4;
#pragma unroll
            for (int ps = 0; ps < PASSES; ++ps)
                *reinterpret_cast<float4 *>(lds + (ps * RPP + rr) * ldk + kq) = r[ps];
        }
    }
};

template <int BM, int BN, int BK, int WM, int WN, int LA, int LB>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64, 2) void gemm_mfma_kernel(GemmParams p)
{
    constexpr int WAVES_N = BN / WN;
    constexpr int NT = (BM / WM) * (BN / WN) * 64;
    constexpr int LDK = BK + 4;
    constexpr int MI = WM / 32, NI = WN / 32;
    static_assert(WM % 32 == 0 && WN % 32 == 0 && BK % 8 == 0, "tile shape");
    using LoadA = TileLoader<LA, BM, BK, NT>;
    using LoadB = TileLoader<LB, BN, BK, NT>;

    __shared__ __attribute__((aligned(16))) float lds[2][(BM + BN) * LDK];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    const unsigned lb = xcd_remap(blockIdx.x, p.total_blocks);
    const unsigned tiles = (unsigned)(p.tiles_m * p.tiles_n);
    const unsigned z = lb / tiles, t_in = lb % tiles;
    const int tile_m = t_in % p.tiles_m, tile_n = t_in / p.tiles_m;
    const int bz = z / p.splits, sp = z % p.splits;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int kb0 = sp * p.kb_per_split;
    const int kb1 = min(p.kbatch, kb0 + p.kb_per_split);

    const float *Ab = p.A + (long long)bz * p.sA;
    const float *Bb = p.B + (long long)bz * p.sB;

    f32x16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    const int kt_per = (p.K + BK - 1) / BK;
    const int n_tiles = (kb1 - kb0) * kt_per;

    float4 ra[LoadA::PASSES], rb[LoadB::PASSES];

    if (n_tiles > 0) {
        LoadA::load(Ab + (long long)kb0 * p.sAk, p.lda, m0, p.M, 0, p.K, tid, ra);
        LoadB::load(Bb + (long long)kb0 * p.sBk, p.ldb, n0, p.N, 0, p.K, tid, rb);
        LoadA::store(lds[0], LDK, tid, ra);
        LoadB::store(lds[0] + BM * LDK, LDK, tid, rb);
    }
    __syncthreads();

    int kb = kb0, kt = 0;
    for (int t = 0; t < n_tiles; ++t) {
        const int cur = t & 1;
        // advance to the next (accumulated batch, k tile) and start fetching it
        if (++kt == kt_per) { kt = 0; ++kb; }
        const bool more = t + 1 < n_tiles;
        if (more) {
            LoadA::load(Ab + (long long)kb * p.sAk, p.lda, m0, p.M, kt * BK, p.K, tid, ra);
            LoadB::load(Bb + (long long)kb * p.sBk, p.ldb, n0, p.N, kt * BK, p.K, tid, rb);
        }

        const float *As = lds[cur] + (wm * WM + (lane & 31)) * LDK + (lane >> 5) * 4;
        const float *Bs = lds[cur] + BM * LDK + (wn * WN + (lane & 31)) * LDK + (lane >> 5) * 4;
#pragma unroll
        for (int kk = 0; kk < BK / 8; ++kk) {
            float4 af[MI], bf[NI];
#pragma unroll
            for (int i = 0; i < MI; ++i) af[i] = *reinterpret_cast<const float4 *>(As + i * 32 * LDK + kk * 8);
#pragma unroll
            for (int j = 0; j < NI; ++j) bf[j] = *reinterpret_cast<const float4 *>(Bs + j * 32 * LDK + kk * 8);
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].x, bf[j].x, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].y, bf[j].y, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].z, bf[j].z, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].w, bf[j].w, acc[i][j], 0, 0, 0);
                }
        }

        if (more) {
            LoadA::store(lds[cur ^ 1], LDK, tid, ra);
            LoadB::store(lds[cur ^ 1] + BM * LDK, LDK, tid, rb);
        }
        __syncthreads();
    }

    // Epilogue.  Accumulator register v of lane l holds row 8*(v/4) + 4*(l/32) + v%4 and column
    // l%32 of its 32x32 block.
    float *Cb;
    long long ldc;
    float alpha, beta;
    if (p.splits > 1) {
        Cb = p.C + (long long)bz * p.sC + (long long)sp * p.sCsplit;
        ldc = p.N;
        alpha = 1.f;
        beta = 0.f;
    } else {
        Cb = p.C + (long long)bz * p.sC;
        ldc = p.ldc;
        alpha = p.alpha;
        beta = p.beta;
    }
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int col = n0 + wn * WN + j * 32 + (lane & 31);
            if (col >= p.N) continue;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = m0 + wm * WM + i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
                if (row < p.M) {
                    float *dst = Cb + (long long)row * ldc + col;
                    const float r = alpha * acc[i][j][v];
                    *dst = beta == 0.f ? r : r + beta * *dst;
                }
            }
        }
}

// C[m][n] = alpha * sum_s partial[s][m][n] + beta * C[m][n], s ascending.
__global__ __launch_bounds__(256) void splitk_fold_kernel(const float *__restrict__ partial, int splits,
                                                          long long split_stride, float *__restrict__ C,
                                                          int M, int N, long long ldc, float alpha,
                                                          float beta)
{
    const long long total = (long long)M * N;
    for (long long e = blockIdx.x * 256LL + threadIdx.x; e < total; e += gridDim.x * 256LL) {
        float acc = 0.f;
        for (int s = 0; s < splits; ++s) acc += partial[s * split_stride + e];
        const int m = (int)(e / N), n = (int)(e - (long long)m * N);
        float *dst = C + m * ldc + n;
        const float r = alpha * acc;
        *dst = beta == 0.f ? r : r + beta * *dst;
    }
}

// ---------------------------------------------------------------------------------------------
// host side: configuration choice and launch
// ---------------------------------------------------------------------------------------------

struct TileCfg {
    int bm, bn;
};

template <int BM, int BN, int BK, int WM, int WN>
static void launch_cfg(hipStream_t st, int la, int lb, const GemmParams &p)
{
    constexpr int NT = (BM / WM) * (BN / WN) * 64;
    const dim3 grid(p.total_blocks), block(NT);
#define AG_GEMM_CASE(LA_, LB_)                                                                        \
    if (la == LA_ && lb == LB_) {                                                                     \
        hipLaunchKernelGGL((gemm_mfma_kernel<BM, BN, BK, WM, WN, LA_, LB_>), grid, block, 0, st, p);  \
        return;                                                                                       \
    }
    AG_GEMM_CASE(LK_VEC, LK_VEC)
    AG_GEMM_CASE(LK_VEC, LK_SCALAR)
    AG_GEMM_CASE(LK_VEC, LMN)
    AG_GEMM_CASE(LK_SCALAR, LK_VEC)
    AG_GEMM_CASE(LK_SCALAR, LK_SCALAR)
    AG_GEMM_CASE(LK_SCALAR, LMN)
    AG_GEMM_CASE(LMN, LK_VEC)
    AG_GEMM_CASE(LMN, LK_SCALAR)
    AG_GEMM_CASE(LMN, LMN)
#undef AG_GEMM_CASE
}

static int g_force_cfg = -1;  // experiment hook, see ag_gemm_force_config

// Tile configurations, largest first.  {BM, BN}; all use BK = 32... except where noted in launch().
static const TileCfg kCfgs[] = {{128, 128}, {128, 64}, {64, 128}, {64, 64}};
constexpr int kNumCfgs = sizeof(kCfgs) / sizeof(kCfgs[0]);

static void launch(hipStream_t st, int cfg, int la, int lb, const GemmParams &p)
{
    switch (cfg) {
        case 0: launch_cfg<128, 128, 32, 64, 64>(st, la, lb, p); break;
        case 1: launch_cfg<128, 64, 32, 64, 32>(st, la, lb, p); break;
        case 2: launch_cfg<64, 128, 32, 32, 64>(st, la, lb, p); break;
        default: launch_cfg<64, 64, 32, 32, 32>(st, la, lb, p); break;
    }
}

static long long cdiv(long long a, long long b) { return (a + b - 1) / b; }

// Pick the configuration with the least padded work, preferring larger tiles on ties, but do
// not starve the 256 CUs: small problems take smaller tiles.
static int choose_cfg(int M, int N, long long zcount)
{
    if (g_force_cfg >= 0 && g_force_cfg < kNumCfgs) return g_force_cfg;
    int best = kNumCfgs - 1;
    double best_cost = 1e300;
    for (int c = 0; c < kNumCfgs; ++c) {
        const long long tm = cdiv(M, kCfgs[c].bm), tn = cdiv(N, kCfgs[c].bn);
        const double blocks = (double)tm * tn * zcount;
        const double tile_work = (double)kCfgs[c].bm * kCfgs[c].bn;
        // waves of 512 resident blocks (2 per CU); partial waves cost a full one
        const double slots = 512.0;
        const double waves = blocks <= slots ? 1.0 : blocks / slots;
        // smaller tiles re-read operands more: penalise them slightly
        const double eff = (c == 0) ? 1.0 : (c == 3 ? 1.25 : 1.1);
        const double cost = waves * tile_work * eff;
        if (cost < best_cost) {
            best_cost = cost;
            best = c;
        }
    }
    return best;
}

static int loader_kind(bool k_contig, const float *ptr, long long ld, int K, long long s1, long long s2)
{
    if (!k_contig) return LMN;
    const bool vec = aligned16(ptr) && ld % 4 == 0 && K % 4 == 0 && s1 % 4 == 0 && s2 % 4 == 0;
    return vec ? LK_VEC : LK_SCALAR;
}

struct GemmCall {
    int transA, transB, M, N, K;
    float alpha, beta;
    const float *A;
    long long lda, sA, sAk;
    const float *B;
    long long ldb, sB, sBk;
    float *C;
    long long ldc, sC;
    int batch, kbatch;
};

static ag_status_t validate(const char *who, const GemmCall &c)
{
    AG_REQUIRE(c.M >= 0 && c.N >= 0 && c.K >= 0 && c.batch >= 0 && c.kbatch >= 0, AG_ERR_INVALID_DIMS,
               "%s: negative extent (M=%d N=%d K=%d batch=%d)", who, c.M, c.N, c.K, c.batch);
    const int a_min = c.transA ? c.M : c.K, b_min = c.transB ? c.K : c.N;
    AG_REQUIRE(c.lda >= (a_min > 1 ? a_min : 1), AG_ERR_INCOMPATIBLE_SHAPE, "%s: lda %lld < %d", who, c.lda, a_min);
    AG_REQUIRE(c.ldb >= (b_min > 1 ? b_min : 1), AG_ERR_INCOMPATIBLE_SHAPE, "%s: ldb %lld < %d", who, c.ldb, b_min);
    AG_REQUIRE(c.ldc >= (c.N > 1 ? c.N : 1), AG_ERR_INCOMPATIBLE_SHAPE, "%s: ldc %lld < %d", who, c.ldc, c.N);
    return AG_OK;
}

// Degenerate K: C = beta*C.
__global__ __launch_bounds__(256) void scale_c_kernel(float *C, int M, int N, long long ldc, long long sC,
                                                      int batch, float beta)
{
    const long long total = (long long)M * N * batch;
    for (long long e = blockIdx.x * 256LL + threadIdx.x; e < total; e += gridDim.x * 256LL) {
        const long long b = e / ((long long)M * N), r = e - b * M * N;
        float *dst = C + b * sC + (r / N) * ldc + (r % N);
        *dst = beta == 0.f ? 0.f : beta * *dst;
    }
}

static ag_status_t run_gemm(hipStream_t st, const char *who, const GemmCall &c, void *ws, size_t ws_bytes,
                            int splits)
{
    if (ag_status_t s = validate(who, c)) return s;
    if (c.M == 0 || c.N == 0 || c.batch == 0) return AG_OK;
    AG_REQUIRE(c.C, AG_ERR_INVALID_DIMS, "%s: null output", who);
    if (c.K == 0 || c.kbatch == 0) {
        const long long total = (long long)c.M * c.N * c.batch;
        hipLaunchKernelGGL(scale_c_kernel, dim3((unsigned)(cdiv(total, 256) > 65536 ? 65536 : cdiv(total, 256))),
                           dim3(256), 0, st, c.C, c.M, c.N, c.ldc, c.sC, c.batch, c.beta);
        return check_launch(who);
    }
    AG_REQUIRE(c.A && c.B, AG_ERR_INVALID_DIMS, "%s: null operand", who);

    GemmParams p;
    p.A = c.A; p.B = c.B; p.C = c.C;
    p.M = c.M; p.N = c.N; p.K = c.K;
    p.lda = c.lda; p.ldb = c.ldb; p.ldc = c.ldc;
    p.sA = c.sA; p.sB = c.sB; p.sC = c.sC;
    p.sAk = c.sAk; p.sBk = c.sBk;
    p.kbatch = c.kbatch;
    p.splits = splits < 1 ? 1 : splits;
    p.kb_per_split = (int)cdiv(c.kbatch, p.splits);
    p.splits = (int)cdiv(c.kbatch, p.kb_per_split);  // drop empty splits
    p.alpha = c.alpha; p.beta = c.beta;
    p.sCsplit = (long long)c.M * c.N;

    const int cfg = choose_cfg(c.M, c.N, (long long)c.batch * p.splits);
    p.tiles_m = (int)cdiv(c.M, kCfgs[cfg].bm);
    p.tiles_n = (int)cdiv(c.N, kCfgs[cfg].bn);
    const long long blocks = (long long)p.tiles_m * p.tiles_n * c.batch * p.splits;
    AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "%s: too many tiles (%lld)", who, blocks);
    p.total_blocks = (unsigned)blocks;

    float *real_c = c.C;
    if (p.splits > 1) {
        const size_t need = sizeof(float) * (size_t)p.splits * c.M * c.N;
        AG_REQUIRE(c.batch == 1, AG_ERR_INVALID_DIMS, "%s: split accumulation with independent batches", who);
        AG_REQUIRE(ws && ws_bytes >= need, AG_ERR_INVALID_DIMS, "%s: workspace of %zu bytes needed, %zu given",
                   who, need, ws_bytes);
        p.C = static_cast<float *>(ws);
    }
    // A is k-contiguous when not transposed; B is k-contiguous when transposed.
    const int la = loader_kind(!c.transA, c.A, c.lda, c.K, c.sA, c.sAk);
    const int lb = loader_kind(c.transB != 0, c.B, c.ldb, c.K, c.sB, c.sBk);
    launch(st, cfg, la, lb, p);
    if (ag_status_t s = check_launch(who)) return s;
    if (p.splits > 1) {
        const long long total = (long long)c.M * c.N;
        hipLaunchKernelGGL(splitk_fold_kernel, dim3((unsigned)(cdiv(total, 256) > 4096 ? 4096 : cdiv(total, 256))),
                           dim3(256), 0, st, static_cast<const float *>(ws), p.splits, p.sCsplit, real_c, c.M,
                           c.N, c.ldc, c.alpha, c.beta);
        return check_launch(who);
    }
    return AG_OK;
}

// Number of splits for an accumulated-batch GEMM: enough blocks for a few waves over the chip.
static int choose_splits(int M, int N, int kbatch)
{
    const int cfg = choose_cfg(M, N, kbatch);  // tile choice as if every image were a block
    const long long tiles = cdiv(M, kCfgs[cfg].bm) * cdiv(N, kCfgs[cfg].bn);
    long long want = cdiv(2048, tiles);
    if (want > kbatch) want = kbatch;
    if (want < 1) want = 1;
    // make the splits even
    const long long per = cdiv(kbatch, want);
    return (int)cdiv(kbatch, per);
}

}  // namespace ag

using namespace ag;

// Experiment hook (not part of the operator surface): force tile configuration `cfg`
// (0..3, -1 = automatic) for subsequent GEMM calls of this process.
extern "C" void ag_gemm_force_config(int cfg) { g_force_cfg = cfg; }

extern "C" ag_status_t ag_gemm_f32(ag_stream_t stream, int transA, int transB, int M, int N, int K,
                                   float alpha, const float *A, int lda, long long strideA, const float *B,
                                   int ldb, long long strideB, float beta, float *C, int ldc,
                                   long long strideC, int batch)
{
    GemmCall c{transA, transB, M, N, K, alpha, beta, A, lda, strideA, 0, B, ldb, strideB, 0, C, ldc, strideC,
               batch, 1};
    return run_gemm(as_stream(stream), "gemm", c, nullptr, 0, 1);
}

extern "C" size_t ag_gemm_batchsum_f32_workspace(int M, int N, int K, int batch)
{
    (void)K;
    if (M <= 0 || N <= 0 || batch <= 0) return 16;
    const int splits = choose_splits(M, N, batch);
    return splits > 1 ? sizeof(float) * (size_t)splits * M * N : 16;
}

extern "C" ag_status_t ag_gemm_batchsum_f32(ag_stream_t stream, int transA, int transB, int M, int N, int K,
                                            float alpha, const float *A, int lda, long long strideA,
                                            const float *B, int ldb, long long strideB, float beta, float *C,
                                            int ldc, int batch, void *ws, size_t ws_bytes)
{
    GemmCall c{transA, transB, M, N, K, alpha, beta, A, lda, 0, strideA, B, ldb, 0, strideB, C, ldc, 0, 1, batch};
    const int splits = (M > 0 && N > 0 && batch > 0) ? choose_splits(M, N, batch) : 1;
    return run_gemm(as_stream(stream), "gemm_batchsum", c, ws, ws_bytes, splits);
}
