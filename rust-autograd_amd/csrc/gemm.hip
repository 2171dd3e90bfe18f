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
#include <mutex>
#include <type_traits>

#ifdef AG_TEST_HOOKS
#include "ag_test_hooks.h"
#endif
#include "gemm_shared.h"

namespace ag {

template <int LT, int ROWS, int BK, int NT>
struct TileLoader {
    static constexpr int QUADS = BK / 4;                 // 4-float groups along k per row
    static constexpr int PASSES = ROWS * QUADS / NT;     // (row, quad) items per thread
    static_assert(ROWS * QUADS % NT == 0 && PASSES >= 1, "tile does not divide over the block");
    static_assert(NT % QUADS == 0, "threads per row must divide the block");

    // Item `it` = ps*NT + tid of this thread.  k-contiguous operands walk the quads of a row with
    // consecutive lanes (128-bit loads along k); mn-contiguous operands walk the rows with
    // consecutive lanes (coalesced 32-bit loads, four k per lane).
    __device__ static inline void item(int it, int &row, int &quad)
    {
        if (LT == LMN) {
            row = it % ROWS;
            quad = it / ROWS;
        } else {
            row = it / QUADS;
            quad = it % QUADS;
        }
    }

    int off[PASSES];   // element offset of this thread's items from the tile origin (row clamped)

    // Offsets are 32-bit (the host checks the operand slice fits) and fixed for the whole k loop:
    // the tile origin moves as a wave-uniform pointer.
    __device__ inline void init(int ld, int row0, int rows, int tid)
    {
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            int rr, q;
            item(ps * NT + tid, rr, q);
            const int row = row0 + rr;
            const int rc = row < rows ? row : rows - 1;
            off[ps] = (LT == LMN) ? q * 4 * ld + rc : rc * ld + q * 4;
        }
    }

    // Distance between the origins of consecutive k tiles.
    __device__ static inline long long k_step(int ld) { return (LT == LMN) ? (long long)BK * ld : BK; }

    // Interior k tile: `origin` = operand + k0 (k-contiguous) or + k0*ld (mn-contiguous).
    __device__ inline void load(const float *__restrict__ origin, int ld, float4 (&r)[PASSES]) const
    {
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            const float *p = origin + off[ps];
            if (LT == LMN) {
                r[ps] = make_float4(p[0], p[ld], p[2 * ld], p[3 * ld]);
            } else if (LT == LK_VEC) {
                r[ps] = *reinterpret_cast<const float4 *>(p);
            } else {
                r[ps] = make_float4(p[0], p[1], p[2], p[3]);
            }
        }
    }

    // Last k tile when K is not a multiple of BK: `krem` (1..BK-1) valid k remain; the rest reads
    // as zero (addresses are clamped, values selected).
    __device__ inline void load_tail(const float *__restrict__ origin, int ld, int krem, int tid,
                                     float4 (&r)[PASSES]) const
    {
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            int rr, q;
            item(ps * NT + tid, rr, q);
            const long long kstride = (LT == LMN) ? ld : 1;
            const float *p = origin + off[ps] - (long long)q * 4 * kstride;   // k = 0 of this row
            float v[4];
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const int k = q * 4 + jj;
                const float x = p[(long long)min(k, krem - 1) * kstride];
                v[jj] = k < krem ? x : 0.f;
            }
            r[ps] = make_float4(v[0], v[1], v[2], v[3]);
        }
    }

    __device__ static inline void store(float *__restrict__ lds, int ldk, int tid, const float4 (&r)[PASSES])
    {
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            int rr, q;
            item(ps * NT + tid, rr, q);
            *reinterpret_cast<float4 *>(lds + rr * ldk + q * 4) = r[ps];
        }
    }
};

template <int BM, int BN, int BK, int WM, int WN, int OCC, int STAGES, int LA, int LB>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64, OCC) void gemm_mfma_kernel(GemmParams p)
{
    static_assert(STAGES == 2 || STAGES == 3, "LDS ring of two or three tiles");
    constexpr int KK = BK / 8;
    constexpr int WAVES_N = BN / WN;
    constexpr int NT = (BM / WM) * (BN / WN) * 64;
    constexpr int LDK = BK + 4;
    constexpr int MI = WM / 32, NI = WN / 32;
    static_assert(WM % 32 == 0 && WN % 32 == 0 && BK % 16 == 0, "tile shape (BK/8 must be even)");
    using LoadA = TileLoader<LA, BM, BK, NT>;
    using LoadB = TileLoader<LB, BN, BK, NT>;

    __shared__ __attribute__((aligned(16))) float lds[STAGES][(BM + BN) * LDK];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    const unsigned total = p.total_blocks;  // work items = tiles x independent batches x splits
    const unsigned tiles = (unsigned)(p.tiles_m * p.tiles_n);
    const int kt_per = (p.K + BK - 1) / BK;
    const int krem = p.K - (kt_per - 1) * BK;  // k in the last tile of a batch
    const bool ktail = krem != BK;
    const int lda = (int)p.lda, ldb = (int)p.ldb;

    // A work item is one output tile of one batch / split.  The block walks items
    // blockIdx.x, blockIdx.x + gridDim.x, ... as ONE stream of k tiles: fetching runs
    // STAGES-1 tiles ahead of the MFMAs and crosses item boundaries, so the loads of the next
    // item are in flight while the current one finishes and is written out.
    struct Item {
        int m0, n0, bz, sp, kb0, nt;
    };
    auto decode = [&](unsigned w) {
        const unsigned lb = xcd_remap(w, total);
        const unsigned z = lb / tiles, t_in = lb % tiles;
        Item it;
        it.m0 = (int)(t_in % p.tiles_m) * BM;
        it.n0 = (int)(t_in / p.tiles_m) * BN;
        it.bz = (int)(z / p.splits);
        it.sp = (int)(z % p.splits);
        it.kb0 = it.sp * p.kb_per_split;
        it.nt = (min(p.kbatch, it.kb0 + p.kb_per_split) - it.kb0) * kt_per;
        return it;
    };

    // ---- fetch stream ----
    unsigned fw = blockIdx.x;
    bool f_valid = fw < total;
    if (!f_valid) return;
    LoadA ldr_a;
    LoadB ldr_b;
    const float *fA = nullptr, *fB = nullptr;
    int fkb = 0, fkt = 0, f_left = 0;
    auto f_begin = [&]() {
        const Item it = decode(fw);
        ldr_a.init(lda, it.m0, p.M, tid);
        ldr_b.init(ldb, it.n0, p.N, tid);
        fA = p.A + (long long)it.bz * p.sA;
        fB = p.B + (long long)it.bz * p.sB;
        fkb = it.kb0;
        fkt = 0;
        f_left = it.nt;
    };
    float4 ra[LoadA::PASSES], rb[LoadB::PASSES];
    // Rows beyond M (or N) are fetched from a clamped, valid address and left as they are: they
    // only feed output rows (columns) that are never written.
    // Loads of the next tile of the stream.  TAIL: K is not a multiple of BK.
    auto fetch_issue = [&](auto tail_tag) {
        const float *oa = fA + (long long)fkb * p.sAk + fkt * LoadA::k_step(lda);
        const float *ob = fB + (long long)fkb * p.sBk + fkt * LoadB::k_step(ldb);
        if (decltype(tail_tag)::value && fkt == kt_per - 1) {
            ldr_a.load_tail(oa, lda, krem, tid, ra);
            ldr_b.load_tail(ob, ldb, krem, tid, rb);
        } else {
            ldr_a.load(oa, lda, ra);
            ldr_b.load(ob, ldb, rb);
        }
    };
    // Move the fetch stream to the following tile (possibly of the next work item).
    // At the end of the stream the position stays on the last tile, which is a valid address for
    // the (discarded) loads issued after it.
    auto fetch_advance = [&]() {
        if (--f_left == 0) {
            fw += gridDim.x;
            f_valid = fw < total;
            if (f_valid) f_begin();
        } else if (++fkt == kt_per) {
            fkt = 0;
            ++fkb;
        }
    };
    auto stage = [&](int buf) {
        LoadA::store(lds[buf], LDK, tid, ra);
        LoadB::store(lds[buf] + BM * LDK, LDK, tid, rb);
    };

    // ---- compute stream ----
    // The MFMAs add to `acc`; after every kChainK elements of k the chain's sum is set aside into
    // `tot` and the chain restarts from zero (see kChainK).
    // Tiles whose two accumulator sets would not fit the register file next to the staged loads
    // (four or more 32 x 32 blocks per wave) keep one chain; long aligned contractions run on the
    // direct-to-LDS kernel, which chains at every tile size.
    constexpr bool CHAINING = MI * NI == 1 || (MI * NI == 2 && OCC <= 2);
    f32x16 acc[MI][NI];
    constexpr int CHAIN = kChainK / BK;  // k tiles per chain
    auto zero_acc = [&]() {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    };
    // Fragment reads: one 128-bit LDS read per 32-row block gives four MFMA k steps.
    const int frag_off = (lane & 31) * LDK + (lane >> 5) * 4;
    auto read_frags = [&](int buf, int kk, float4 (&af)[MI], float4 (&bf)[NI]) {
        const float *As = lds[buf] + wm * WM * LDK + frag_off + kk * 8;
        const float *Bs = lds[buf] + (BM + wn * WN) * LDK + frag_off + kk * 8;
#pragma unroll
        for (int i = 0; i < MI; ++i) af[i] = *reinterpret_cast<const float4 *>(As + i * 32 * LDK);
#pragma unroll
        for (int j = 0; j < NI; ++j) bf[j] = *reinterpret_cast<const float4 *>(Bs + j * 32 * LDK);
    };
    auto mfma_frags = [&](const float4 (&af)[MI], const float4 (&bf)[NI]) {
        // k step outermost: consecutive MFMAs write different accumulators
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j) {
                    const float a = s4 == 0 ? af[i].x : s4 == 1 ? af[i].y : s4 == 2 ? af[i].z : af[i].w;
                    const float b = s4 == 0 ? bf[j].x : s4 == 1 ? bf[j].y : s4 == 2 ? bf[j].z : bf[j].w;
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i][j], 0, 0, 0);
                }
    };
    // Accumulator register v of lane l holds row 8*(v/4) + 4*(l/32) + v%4 and column l%32 of its
    // 32x32 block.
    auto write_out = [&](const Item &it) {
        float *Cb;
        long long ldc;
        float alpha, beta;
        if (p.splits > 1) {
            Cb = p.C + (long long)it.bz * p.sC + (long long)it.sp * p.sCsplit;
            ldc = p.N;
            alpha = 1.f;
            beta = 0.f;
        } else {
            Cb = p.C + (long long)it.bz * p.sC;
            ldc = p.ldc;
            alpha = p.alpha;
            beta = p.beta;
        }
        const bool full = it.m0 + BM <= p.M && it.n0 + BN <= p.N;
        const int row_base = it.m0 + wm * WM + 4 * (lane >> 5);
        const int col_base = it.n0 + wn * WN + (lane & 31);
        if (full && beta == 0.f) {
            // interior tile, overwrite: straight stores
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j) {
                    float *dst = Cb + (long long)(row_base + i * 32) * ldc + col_base + j * 32;
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        dst[(long long)(8 * (v / 4) + (v % 4)) * ldc] = alpha * acc[i][j][v];
                }
        } else {
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j) {
                    const int col = col_base + j * 32;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int row = row_base + i * 32 + 8 * (v / 4) + (v % 4);
                        if (row < p.M && col < p.N) {
                            float *dst = Cb + (long long)row * ldc + col;
                            const float r = alpha * acc[i][j][v];
                            *dst = beta == 0.f ? r : r + beta * *dst;
                        }
                    }
                }
        }
    };

    auto run = [&](auto tail_tag) __attribute__((always_inline)) {
        // Prologue: the first STAGES-1 tiles of the stream go to LDS.
        f_begin();
#pragma unroll
        for (int st = 0; st < STAGES - 1; ++st)
            if (f_valid) {
                fetch_issue(tail_tag);
                fetch_advance();
                stage(st);
            }
        __syncthreads();

        unsigned cw = blockIdx.x;
        Item ci = decode(cw);
        int c_left = ci.nt;
        zero_acc();
        // (plain loops, not lambdas: a further closure level keeps the arrays from being promoted to registers)
        f32x16 tot[CHAINING ? MI : 1][CHAINING ? NI : 1];
#define AG_FOR_TOT(stmt)                                       \
    if constexpr (CHAINING) {                                  \
        _Pragma("unroll") for (int i = 0; i < MI; ++i)         \
        _Pragma("unroll") for (int j = 0; j < NI; ++j)         \
        _Pragma("unroll") for (int v = 0; v < 16; ++v) { stmt; } \
    }
        bool chained = CHAINING && ci.nt > CHAIN + CHAIN / 4;  // more than one chain: their sums meet in `tot`
        if (chained) AG_FOR_TOT(tot[i][j][v] = 0.f)
        int chain_left = CHAIN;
        float4 af[2][MI], bf[2][NI];
        read_frags(0, 0, af[0], bf[0]);

        int cur = 0;                       // ring slot of the tile being multiplied
        int fill = (STAGES - 1) % STAGES;  // ring slot the tile being fetched goes to
        while (true) {
            const bool more = f_valid;
            if (more) fetch_issue(tail_tag);  // global loads fly during this tile's MFMAs
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                if (kk + 1 < KK) read_frags(cur, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
                mfma_frags(af[kk & 1], bf[kk & 1]);
            }
            if (more) {
                fetch_advance();
                stage(fill);
            }
            const bool item_done = --c_left == 0;
            const bool last = item_done && cw + gridDim.x >= total;  // nothing follows in the stream
            const int nxt = cur + 1 == STAGES ? 0 : cur + 1;
            if (STAGES == 3) {
                // The next tile was completed before the previous barrier: start reading it now.
                if (!last) read_frags(nxt, 0, af[0], bf[0]);
                __syncthreads();
            } else {
                __syncthreads();
                if (!last) read_frags(nxt, 0, af[0], bf[0]);
            }
            cur = nxt;
            fill = fill + 1 == STAGES ? 0 : fill + 1;

            if (item_done) {
                if (chained) AG_FOR_TOT(acc[i][j][v] += tot[i][j][v])
                write_out(ci);
                if (last) break;
                cw += gridDim.x;
                ci = decode(cw);
                c_left = ci.nt;
                zero_acc();
                chained = CHAINING && ci.nt > CHAIN + CHAIN / 4;
                if (chained) AG_FOR_TOT(tot[i][j][v] = 0.f)
                chain_left = CHAIN;
            } else if (CHAINING && --chain_left == 0 && c_left > CHAIN / 4) {
                // (a remainder of up to a quarter chain joins the chain before it)
                AG_FOR_TOT(tot[i][j][v] += acc[i][j][v]; acc[i][j][v] = 0.f)
                chain_left = CHAIN;
            }
        }
    };
    if (ktail) run(std::true_type{});
    else run(std::false_type{});
#undef AG_FOR_TOT
}

// C[m][n] = alpha * sum_s partial[s][m][n] + beta * C[m][n].  A block folds 32 consecutive
// elements: thread (g, e) adds the partials s = g, g + 8, g + 16, ... of element e (eight
// independent chains keep enough loads in flight), then the eight group sums are added in
// ascending g.  The order is fixed, so the result is deterministic.
__global__ __launch_bounds__(256) void splitk_fold_kernel(const float *__restrict__ partial, int splits,
                                                          long long split_stride, float *__restrict__ C,
                                                          int M, int N, long long ldc, float alpha,
                                                          float beta)
{
    __shared__ float part[8][32];
    const long long total = (long long)M * N;
    const int e_in = threadIdx.x & 31, grp = threadIdx.x >> 5;
    for (long long e0 = blockIdx.x * 32LL; e0 < total; e0 += gridDim.x * 32LL) {
        const long long e = e0 + e_in;
        float acc = 0.f;
        if (e < total)
            for (int s = grp; s < splits; s += 8) acc += partial[s * split_stride + e];
        part[grp][e_in] = acc;
        __syncthreads();
        if (grp == 0 && e < total) {
            float sum = part[0][e_in];
#pragma unroll
            for (int g = 1; g < 8; ++g) sum += part[g][e_in];
            const int m = (int)(e / N), n = (int)(e - (long long)m * N);
            float *dst = C + m * ldc + n;
            const float r = alpha * sum;
            *dst = beta == 0.f ? r : r + beta * *dst;
        }
        __syncthreads();
    }
}

// The same fold over four consecutive elements per thread (128 per block) with 128-bit loads, four
// of them in flight per chain: per element the additions are the ones of splitk_fold_kernel in the
// same order, so the two kernels give identical results.  Needs total, split_stride and N
// multiples of four, ldc a multiple of four and 16-byte aligned partials and C.
__global__ __launch_bounds__(256) void splitk_fold_vec_kernel(const float *__restrict__ partial, int splits,
                                                              long long split_stride, float *__restrict__ C,
                                                              int M, int N, long long ldc, float alpha,
                                                              float beta)
{
    __shared__ float4 part[8][32];
    const long long quads = (long long)M * N / 4, stride4 = split_stride / 4;
    const float4 *p4 = reinterpret_cast<const float4 *>(partial);
    const int q_in = threadIdx.x & 31, grp = threadIdx.x >> 5;
    for (long long q0 = blockIdx.x * 32LL; q0 < quads; q0 += gridDim.x * 32LL) {
        const long long q = q0 + q_in;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        if (q < quads) {
            int sidx = grp;
            for (; sidx + 24 < splits; sidx += 32) {
                float4 v[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) v[u] = p4[(sidx + 8 * u) * stride4 + q];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    acc.x += v[u].x;
                    acc.y += v[u].y;
                    acc.z += v[u].z;
                    acc.w += v[u].w;
                }
            }
            for (; sidx < splits; sidx += 8) {
                const float4 v = p4[sidx * stride4 + q];
                acc.x += v.x;
                acc.y += v.y;
                acc.z += v.z;
                acc.w += v.w;
            }
        }
        part[grp][q_in] = acc;
        __syncthreads();
        if (grp == 0 && q < quads) {
            float4 sum = part[0][q_in];
#pragma unroll
            for (int g = 1; g < 8; ++g) {
                sum.x += part[g][q_in].x;
                sum.y += part[g][q_in].y;
                sum.z += part[g][q_in].z;
                sum.w += part[g][q_in].w;
            }
            const long long e = q * 4;
            const int m = (int)(e / N), n = (int)(e - (long long)m * N);
            float4 *dst = reinterpret_cast<float4 *>(C + m * ldc + n);
            float4 r = make_float4(alpha * sum.x, alpha * sum.y, alpha * sum.z, alpha * sum.w);
            if (beta != 0.f) {
                const float4 old = *dst;
                r.x += beta * old.x;
                r.y += beta * old.y;
                r.z += beta * old.z;
                r.w += beta * old.w;
            }
            *dst = r;
        }
        __syncthreads();
    }
}

// Launches the fold that suits the operands.
static void launch_fold(hipStream_t st, const float *ws, int splits, long long split_stride, float *C, int M, int N,
                        long long ldc, float alpha, float beta)
{
    const long long total = (long long)M * N;
    const bool vec = total % 4 == 0 && N % 4 == 0 && ldc % 4 == 0 && split_stride % 4 == 0 && aligned16(ws) && aligned16(C);
    if (vec) {
        const long long blocks = (total / 4 + 31) / 32;
        hipLaunchKernelGGL(splitk_fold_vec_kernel, dim3((unsigned)(blocks > 16384 ? 16384 : blocks)), dim3(256), 0, st, ws,
                           splits, split_stride, C, M, N, ldc, alpha, beta);
    } else {
        const long long blocks = (total + 31) / 32;
        hipLaunchKernelGGL(splitk_fold_kernel, dim3((unsigned)(blocks > 16384 ? 16384 : blocks)), dim3(256), 0, st, ws,
                           splits, split_stride, C, M, N, ldc, alpha, beta);
    }
}

// ---------------------------------------------------------------------------------------------
// host side: configuration choice and launch
// ---------------------------------------------------------------------------------------------

struct TileCfg {
    int bm, bn;
};

// Resident blocks per CU of one kernel instantiation, and the CU count (both cached).
static int num_cus() { return device_cus(); }

// Blocks of the direct-to-LDS kernel's persistent grid: one per CU, a multiple of the XCD count.
static long long direct_grid(int cus) { return cus >= kXcds ? cus - cus % kXcds : kXcds; }

template <typename Kern>
static int resident_blocks(Kern kern, int threads, int fallback)
{
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, threads, 0) != hipSuccess || n < 1) n = fallback;
    return n;
}

// Test hooks (ag_test_hooks.h; built only into the test flavour of the library, -DAG_TEST_HOOKS), per calling
// thread: blocks per CU of the persistent grid (0 = resident count), a forced tile configuration (-1 = automatic
// choice) and a forced split count of accumulated-batch products (0 = automatic).
#ifdef AG_TEST_HOOKS
static thread_local int g_grid_scale = 0;
static thread_local int g_force_cfg = -1;
static thread_local int g_force_splits = 0;
#else
constexpr int g_grid_scale = 0, g_force_cfg = -1, g_force_splits = 0;
#endif

template <int BM, int BN, int BK, int WM, int WN, int OCC, int STAGES>
static void launch_cfg(hipStream_t st, int la, int lb, const GemmParams &p)
{
    constexpr int NT = (BM / WM) * (BN / WN) * 64;
    const dim3 block(NT);
#define AG_GEMM_CASE(LA_, LB_)                                                                        \
    if (la == LA_ && lb == LB_) {                                                                     \
        auto kern = gemm_mfma_kernel<BM, BN, BK, WM, WN, OCC, STAGES, LA_, LB_>;                      \
        static const int per_cu = resident_blocks(kern, NT, OCC);                                     \
        /* persistent grid: every resident slot gets one block, which walks the items */             \
        long long g = (long long)num_cus() * (g_grid_scale > 0 ? g_grid_scale : per_cu);              \
        if (g > p.total_blocks) g = p.total_blocks;                                                   \
        hipLaunchKernelGGL(kern, dim3((unsigned)g), block, 0, st, p);                                 \
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

// Tile configurations {BM, BN}; see launch() for BK, the wave tile and the occupancy target.
static const TileCfg kCfgs[] = {{128, 128}, {128, 64}, {64, 128}, {64, 64},
                                {128, 128}, {192, 128}, {256, 128}, {128, 256}, {64, 64}, {128, 64},
                                {128, 128}, {192, 128}, {128, 64},
                                {128, 128}, {128, 256}, {256, 128}, {192, 128}, {128, 192}, {128, 64}, {64, 128},
                                {32, 128}, {64, 64}};
constexpr int kNumCfgs = sizeof(kCfgs) / sizeof(kCfgs[0]);
static void launch(hipStream_t st, int cfg, int la, int lb, const GemmParams &p)
{
    switch (cfg) {
        //                 BM   BN  BK  WM   WN OCC STAGES
        case 0: launch_cfg<128, 128, 32, 64, 64, 2, 2>(st, la, lb, p); break;
        case 1: launch_cfg<128, 64, 32, 64, 32, 2, 2>(st, la, lb, p); break;
        case 2: launch_cfg<64, 128, 32, 32, 64, 2, 2>(st, la, lb, p); break;
        case 3: launch_cfg<64, 64, 32, 32, 32, 2, 2>(st, la, lb, p); break;
        case 4: launch_cfg<128, 128, 16, 64, 64, 3, 2>(st, la, lb, p); break;
        case 5: launch_cfg<192, 128, 16, 96, 64, 2, 2>(st, la, lb, p); break;
        case 6: launch_cfg<256, 128, 16, 128, 64, 2, 2>(st, la, lb, p); break;
        case 7: launch_cfg<128, 256, 16, 64, 128, 2, 2>(st, la, lb, p); break;
        case 8: launch_cfg<64, 64, 16, 32, 32, 4, 2>(st, la, lb, p); break;
        case 9: launch_cfg<128, 64, 16, 64, 32, 3, 2>(st, la, lb, p); break;
        case 10: launch_cfg<128, 128, 16, 64, 64, 2, 3>(st, la, lb, p); break;
        case 11: launch_cfg<192, 128, 16, 96, 64, 2, 3>(st, la, lb, p); break;
        default: launch_cfg<128, 64, 16, 64, 32, 3, 3>(st, la, lb, p); break;
    }
}

static long long cdiv(long long a, long long b) { return (a + b - 1) / b; }

// Tile choice.  The block-tile shape comes first: least padded output area, larger tiles on ties
// (they re-read operands less).  Problems the direct-to-LDS kernel accepts (`direct`) choose among
// its five tiles; the eight-wave tiles keep the matrix pipe about 8 % busier than the four-wave
// 128 x 128 tile, which is weighed against their padding.  Otherwise: contractions with few k
// tiles per output tile, and the accumulated-batch GEMMs, take the BK = 16 family with a
// three-tile LDS ring, long contractions take BK = 32.  Problems too small to give every CU a
// block fall back to 64 x 64 tiles of the register-staged kernel.
// `tail_split`: the launch will be cut into whole rounds plus a narrow-tile tail (folded batch with
// one row of tiles), so a partly filled last round costs nothing here.
// `a_kcontig`: A is k-contiguous (not transposed), which the 32-row tile needs.
static int choose_cfg(int M, int N, int K, long long zcount, bool accumulate, bool direct, bool tail_split = false,
                      bool a_kcontig = false)
{
    if (g_force_cfg >= 0 && g_force_cfg < kNumCfgs) return g_force_cfg == kDirectCfg32 && !a_kcontig ? kDirectCfg64 : g_force_cfg;
    if (direct) {
        // 128x256, 256x128, 192x128, 128x192, 128x128, and 64x128 / 64x64 (two blocks per CU); the efficiencies are
        // what each tile reaches on 6144^3, where every one of them has whole rounds (144 TFLOP/s = 1)
        static const int dl[] = {14, 15, 16, 17, 13, kDirectCfg64, kDirectCfg64Narrow};
        static const double eff[] = {1.0, 1.0, 0.98, 0.98, 0.93, 0.95, 0.89};
        constexpr int kCandidates = 7;
        // The cheapest tile among those that give the chip at least half a round of blocks: padded
        // area over efficiency, counted in whole rounds of the persistent grid while there are few
        // of them (264 blocks on 256 CUs take two rounds, 200 take one).
        // up to 64 (32) output rows: taller tiles would spend half of their matrix work on padding; a
        // problem that gives the chip fewer than two 64 x 128 blocks per CU takes 64 x 64 tiles instead
        const long long wide = cdiv(N, 128) * zcount, cus2 = direct_grid(num_cus());
        if (M <= 32 && a_kcontig && wide >= cus2 / 2) return kDirectCfg32;
        if (M <= 64 && wide >= cus2 / 2) return wide < 2 * cus2 ? kDirectCfg64Narrow : kDirectCfg64;
        // fewer 128 x 128 tiles than CUs: 64 x 64 tiles (two or three blocks per CU) use the whole chip
        if (!accumulate && cdiv(M, 128) * cdiv(N, 128) * zcount < cus2 && cdiv(M, 64) * cdiv(N, 64) * zcount >= cus2 / 2)
            return kDirectCfg64Narrow;
        // a short contraction over a few rounds of tiles: the prologue and epilogue of a tile weigh as much as
        // its k loop, and two 64 x 128 blocks per CU overlap the one's with the other's (M = 2304, N = 32 x 196,
        // K = 256: 71 us against 89 us with 256 x 128 tiles)
        if (!accumulate && K <= 512 && M >= 64 && cdiv(M, 128) * cdiv(N, 128) * zcount < 8 * cus2) return kDirectCfg64;
        int best = -1;
        double best_cost = 1e300;
        for (int c = 0; c < kCandidates; ++c) {
            const TileCfg &t = kCfgs[dl[c]];
            const long long tm = cdiv(M, t.bm), tn = cdiv(N, t.bn);
            const long long blocks = tm * tn * zcount;
            const long long grid = direct_grid(num_cus()) * (t.bm == 64 ? 2 : 1);
            if (blocks < direct_grid(num_cus()) / 2) continue;
            const bool whole_rounds = blocks < 8 * grid && !(tail_split && t.bm == 128 && tm == 1);
            const long long counted = whole_rounds ? cdiv(blocks, grid) * grid : blocks;
            // equal round counts: the tile with less padding wins
            const double padding = (double)tm * t.bm * tn * t.bn / ((double)M * N) - 1.0;
            const double cost = (double)counted * t.bm * t.bn / zcount / eff[c] * (1.0 + 0.5 * padding);
            if (cost < best_cost * 0.995) {
                best_cost = cost;
                best = dl[c];
            }
        }
        if (best >= 0) return best;
    }
    static const int short_k[] = {11, 10, 12, 8};  // 192x128, 128x128, 128x64, 64x64 (BK 16)
    static const int long_k[] = {0, 1, 2, 3};      // 128x128, 128x64, 64x128, 64x64 (BK 32)
    const bool use_short = accumulate || K <= 1024;
    const int *cand = use_short ? short_k : long_k;
    int best = cand[3];
    double best_area = 1e300;
    long long best_blocks = 0;
    for (int c = 0; c < 4; ++c) {
        const TileCfg &t = kCfgs[cand[c]];
        const long long tm = cdiv(M, t.bm), tn = cdiv(N, t.bn);
        const double area = (double)tm * t.bm * tn * t.bn;
        if (area < best_area * 0.97) {  // needs a >3 % saving to beat a larger tile
            best_area = area;
            best = cand[c];
            best_blocks = tm * tn * zcount;
        }
    }
    if (best_blocks < 256) best = cand[3];
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

// What the direct-to-LDS kernel asks of the operands' layout (their size apart).
static bool direct_layout_ok(const GemmCall &c)
{
    auto mult4 = [](long long v) { return v % 4 == 0; };
    if (c.K % 32 != 0 || !aligned16(c.A) || !aligned16(c.B)) return false;
    if (!mult4(c.lda) || !mult4(c.ldb) || !mult4(c.sA) || !mult4(c.sB) || !mult4(c.sAk) || !mult4(c.sBk)) return false;
    if (c.transA && (c.M % 4 != 0 || c.M < 4)) return false;   // A is m-contiguous
    if (!c.transB && (c.N % 4 != 0 || c.N < 4)) return false;  // B is n-contiguous
    return true;
}

static bool direct_ok(const GemmCall &c)
{
    if (!direct_layout_ok(c)) return false;
    // byte offsets inside one operand slice are unsigned 32-bit
    const long long a_span = c.transA ? (long long)(c.K - 1) * c.lda + c.M : (long long)(c.M - 1) * c.lda + c.K;
    const long long b_span = c.transB ? (long long)(c.N - 1) * c.ldb + c.K : (long long)(c.K - 1) * c.ldb + c.N;
    return a_span < (1LL << 30) && b_span < (1LL << 30);
}

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

// `partials_only` >= 0 (split accumulations only): the partial sums are written from split slot
// `partials_only` of the workspace onwards and left for the caller to fold; `*used_splits` receives
// their number.
static ag_status_t run_gemm(hipStream_t st, const char *who, const GemmCall &c, void *ws, size_t ws_bytes,
                            int splits, int partials_only = -1, int *used_splits = nullptr)
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
    // Tile offsets inside one operand slice are 32-bit: element offsets in the register-staged kernel, byte
    // offsets in the direct-to-LDS kernel.  A single product with an operand of 2^31 elements or more (2^30 where
    // the layout suits the direct-to-LDS kernel, so that large products stay on it: 32768^3 is four launches of
    // 16384 x 32768 x 16384) is cut in two until the pieces fit: along that operand's own rows where they are rows
    // or columns of the output (two independent products), else along k (the second piece accumulates on top of
    // the first).
    if (c.kbatch == 1 && partials_only < 0) {
        const long long lim = direct_layout_ok(c) && c.K >= 64 ? (1LL << 30) : 0x7fffffffLL;
        const long long a_all = c.transA ? (long long)(c.K - 1) * c.lda + c.M : (long long)(c.M - 1) * c.lda + c.K;
        const long long b_all = c.transB ? (long long)(c.N - 1) * c.ldb + c.K : (long long)(c.K - 1) * c.ldb + c.N;
        if (a_all >= lim || b_all >= lim) {
            auto half = [](int n) { return n >= 512 ? n / 2 - (n / 2) % 256 : n / 2; };  // keeps tiles and alignment whole
            GemmCall lo = c, hi = c;
            bool cut = true;
            if (a_all >= lim && !c.transA && c.M > 1) {
                lo.M = half(c.M);
                hi.M = c.M - lo.M;
                hi.A = c.A + (long long)lo.M * c.lda;
                hi.C = c.C + (long long)lo.M * c.ldc;
            } else if (b_all >= lim && c.transB && c.N > 1) {
                lo.N = half(c.N);
                hi.N = c.N - lo.N;
                hi.B = c.B + (long long)lo.N * c.ldb;
                hi.C = c.C + lo.N;
            } else if (c.K > 1) {
                lo.K = half(c.K);
                hi.K = c.K - lo.K;
                hi.beta = 1.f;
                hi.A = c.A + (c.transA ? (long long)lo.K * c.lda : (long long)lo.K);
                hi.B = c.B + (c.transB ? (long long)lo.K : (long long)lo.K * c.ldb);
            } else {
                cut = false;  // one row or column longer than 2^31: refused below
            }
            if (cut) {
                if (ag_status_t s = run_gemm(st, who, lo, ws, ws_bytes, splits)) return s;
                return run_gemm(st, who, hi, ws, ws_bytes, splits);
            }
        }
    }
    // A long contraction that misses the direct-to-LDS kernel only because K is not a multiple of
    // its k tile: the whole tiles go there, the remaining K % 32 are accumulated on top by the
    // register-staged kernel (2-3 % of the work).  A single product shorter than 1024 does so only while its
    // output is small: the second pass reads and writes C once more (1000^3: 55 -> 40 us; 4096 x 4096 x 520 would
    // go from 170 to 223 us).
    const bool worth_two_passes = c.kbatch > 1 || c.K >= 1024 || (c.K >= 512 && (long long)c.M * c.N <= 2500000);
    if (c.K % 32 != 0 && c.K >= 256 && worth_two_passes && g_force_cfg < 0 && !direct_ok(c)) {
        GemmCall body = c;
        body.K = c.K - c.K % 32;
        // only when the body really lands on the direct-to-LDS kernel (enough tiles for it)
        const int eff_splits = splits < 1 ? 1 : (int)cdiv(c.kbatch, cdiv(c.kbatch, splits));
        if (direct_ok(body) &&
            choose_cfg(body.M, body.N, body.K, (long long)body.batch * eff_splits, body.kbatch > 1, true, false, !body.transA) >=
                kFirstDirectCfg) {
            GemmCall rest = c;
            rest.K = c.K % 32;
            rest.beta = 1.f;
            rest.A = c.A + (c.transA ? (long long)body.K * c.lda : (long long)body.K);
            rest.B = c.B + (c.transB ? (long long)body.K : (long long)body.K * c.ldb);
            const size_t slot = sizeof(float) * (size_t)c.M * c.N;
            if (splits > 1 && partials_only < 0 && c.batch == 1 && ws && ws_bytes >= 2 * (size_t)splits * slot) {
                // both passes leave their partial sums side by side; one fold adds them all
                int s_body = 0, s_rest = 0;
                if (ag_status_t s = run_gemm(st, who, body, ws, ws_bytes, splits, 0, &s_body)) return s;
                if (s_body <= 1) {  // the body did not split after all and has written C
                    rest.beta = 1.f;
                    return run_gemm(st, who, rest, ws, ws_bytes, splits);
                }
                rest.beta = c.beta;
                // the tail is a few per cent of the work: an eighth of the splits keeps its partial sums small
                if (ag_status_t s = run_gemm(st, who, rest, ws, ws_bytes, splits >= 16 ? splits / 8 : 2, s_body, &s_rest)) return s;
                // rest split: fold everything onto beta * C; rest not split: it has written
                // alpha * rest + beta * C, the body's partial sums are added on top
                const long long total = (long long)c.M * c.N;
                launch_fold(st, static_cast<const float *>(ws), s_rest > 1 ? s_body + s_rest : s_body, total, c.C, c.M, c.N,
                            c.ldc, c.alpha, s_rest > 1 ? c.beta : 1.f);
                return check_launch(who);
            }
            if (ag_status_t s = run_gemm(st, who, body, ws, ws_bytes, splits)) return s;
            return run_gemm(st, who, rest, ws, ws_bytes, splits);
        }
    }
    // tile offsets inside one operand slice are 32-bit
    const long long a_span = c.transA ? (long long)(c.K - 1) * c.lda + c.M : (long long)(c.M - 1) * c.lda + c.K;
    const long long b_span = c.transB ? (long long)(c.N - 1) * c.ldb + c.K : (long long)(c.K - 1) * c.ldb + c.N;
    AG_REQUIRE(a_span < 0x7fffffffLL && b_span < 0x7fffffffLL, AG_ERR_INVALID_DIMS,
               "%s: an operand slice spans %lld elements; at most 2^31-1 supported", who,
               a_span > b_span ? a_span : b_span);

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

    // Independent batches that share A and are n-contiguous in B and C can be laid side by side
    // along n (direct-to-LDS kernel): N = batch * n is then tiled without padding every batch.
    const bool foldable = direct_ok(c) && c.batch > 1 && p.splits == 1 && c.kbatch == 1 && c.sA == 0 &&
                          !c.transB && c.N % 4 == 0 && (long long)c.N * c.batch < 0x7fffffffLL &&
                          c.sB < (1LL << 30) && c.sB % 4 == 0;
    int cfg = choose_cfg(c.M, foldable ? c.N * c.batch : c.N, c.K, foldable ? 1 : (long long)c.batch * p.splits,
                         c.kbatch > 1, direct_ok(c), foldable && g_force_cfg < 0, !c.transA);
    if (cfg >= kFirstDirectCfg && !direct_ok(c)) cfg = 0;  // a forced configuration that cannot run
    const bool fold = foldable && cfg >= kFirstDirectCfg && c.N >= kCfgs[cfg].bn;
    p.n_img = fold ? c.N : 0;
    if (fold) p.N = c.N * c.batch;
    p.n_off = 0;
    p.conv_wp = p.conv_w = p.conv_kw = 0;
    p.conv_pair_w = p.conv_pair_a = 0;
    p.conv_pair_grouped = 0;
    p.conv_pair_skip[0] = p.conv_pair_skip[1] = 0;
    p.conv_phase = 0;
    p.conv_dil = 1;
    p.rows_taps = p.rows_kw = p.rows_wp = 0;
    p.rows_plane = p.rows_phase = 0;
    p.tiles_m = (int)cdiv(c.M, kCfgs[cfg].bm);
    p.tiles_n = (int)cdiv(p.N, kCfgs[cfg].bn);
    const long long blocks = (long long)p.tiles_m * p.tiles_n * (fold ? 1 : c.batch) * p.splits;
    AG_REQUIRE(blocks <= kMaxGridX, AG_ERR_INVALID_DIMS, "%s: too many tiles (%lld)", who, blocks);
    p.total_blocks = (unsigned)blocks;

    // A persistent grid of G blocks takes ceil(items / G) rounds; when the last round would be
    // mostly idle (12.25 rounds at the headline forward shape) the folded problem is cut in two
    // launches: whole rounds of the chosen tile, then the remaining columns with a narrower tile
    // (128 x 64 or 128 x 128) that fills the chip once more for a fraction of a round.
    int tail_cfg = -1;
    GemmParams tail = p;
    if (fold && g_force_cfg < 0 && kCfgs[cfg].bm == 128 && p.tiles_m == 1) {
        const long long G = direct_grid(num_cus());
        const long long rounds = blocks / G, rem = blocks % G;
        if (rounds >= 1 && rem > 0) {
            const int bn = kCfgs[cfg].bn;
            const long long main_cols = rounds * G * bn;
            double best = (double)rounds + 1.0 - 0.05;
            static const int narrow[] = {18, 13};  // 128 x 64, 128 x 128
            static const double eff[] = {0.85, 0.92};
            for (int t = 0; t < 2; ++t) {
                const int bnt = kCfgs[narrow[t]].bn;
                if (bnt >= bn) continue;
                const long long items = cdiv(p.N - main_cols, bnt);
                const double cost = (double)rounds + (double)cdiv(items, G) * bnt / bn / eff[t];
                if (cost < best) {
                    best = cost;
                    tail_cfg = narrow[t];
                }
            }
            if (tail_cfg >= 0) {
                tail.n_off = (int)main_cols;
                tail.tiles_n = (int)cdiv(p.N - main_cols, kCfgs[tail_cfg].bn);
                tail.total_blocks = (unsigned)tail.tiles_n;
                p.N = (int)main_cols;
                p.tiles_n = (int)(rounds * G);
                p.total_blocks = (unsigned)p.tiles_n;
            }
        }
    }

    float *real_c = c.C;
    if (used_splits) *used_splits = p.splits;
    const int first_slot = partials_only > 0 ? partials_only : 0;
    if (p.splits > 1) {
        const size_t need = sizeof(float) * (size_t)(first_slot + p.splits) * c.M * c.N;
        AG_REQUIRE(c.batch == 1, AG_ERR_INVALID_DIMS, "%s: split accumulation with independent batches", who);
        AG_REQUIRE(ws && ws_bytes >= need, AG_ERR_INVALID_DIMS, "%s: workspace of %zu bytes needed, %zu given",
                   who, need, ws_bytes);
        p.C = static_cast<float *>(ws) + (size_t)first_slot * c.M * c.N;
    }
    // A is k-contiguous when not transposed; B is k-contiguous when transposed.
    const int la = loader_kind(!c.transA, c.A, c.lda, c.K, c.sA, c.sAk);
    const int lb = loader_kind(c.transB != 0, c.B, c.ldb, c.K, c.sB, c.sBk);
    if (cfg >= kFirstDirectCfg) launch_direct(st, cfg, !c.transA, c.transB != 0, p, num_cus(), g_grid_scale);
    else launch(st, cfg, la, lb, p);
    if (ag_status_t s = check_launch(who)) return s;
    if (tail_cfg >= 0) {
        launch_direct(st, tail_cfg, !c.transA, c.transB != 0, tail, num_cus(), g_grid_scale);
        if (ag_status_t s = check_launch(who)) return s;
    }
    if (p.splits > 1 && partials_only < 0) {
        launch_fold(st, static_cast<const float *>(ws), p.splits, p.sCsplit, real_c, c.M, c.N, c.ldc, c.alpha, c.beta);
        return check_launch(who);
    }
    return AG_OK;
}

// Implicit input gradient of a stride-1 convolution on the direct-to-LDS kernel (see the conv_*
// fields of GemmParams): gx[b][c] = sum over taps and filters of wr[c][tap][k] * gyp[b][k] shifted.
// wr [C][kh*kw*Kf] (k fastest), gyp [B][Kf][Hp][Wp] zero-bordered, gx [B][C][H][W].
// `phase` != 0: stride-2 forward over four phase planes of `phase` elements per contracted channel.
// `pair_w` != 0: the pair form of the stride-2 input gradient (C counts the 2 x channels rows; the output planes are
// pair_h x pair_w and receive row parity pair_a).
// Tile and split of one implicit convolution product (M = C output rows, N = B * H * Wp padded columns, contraction
// over taps x Kf).  `splits` > 1: the walk over the Kf / 32 channel groups is cut into that many ranges whose partial
// results (each laid out like the output) a fixed-order fold adds up -- for products with fewer tiles than the chip
// has room for, where a slice of the contraction per block keeps every CU busy.
struct ImplicitPlan {
    int cfg, splits;
};
static ImplicitPlan implicit_plan(int B, int C, int Kf, int H, int Wp, int taps, unsigned phase, int pair_w, bool may_split);

// What conv_implicit_gemm launches: a product on tile `cfg`, then, if tail_cfg >= 0, its last columns on a narrower one.
struct ImplicitLaunch {
    GemmParams p, tail;
    int cfg, tail_cfg;
};

// `plan_only` != null: nothing is launched, the launches are described there instead (for a caller that merges two
// products into one launch).
static ag_status_t conv_implicit_gemm(hipStream_t st, const float *wr, const float *gyp, float *gx, int B, int C, int Kf,
                                      int H, int W, int kh, int kw, int Hp, int Wp, unsigned phase, int pair_w = 0,
                                      int pair_a = 0, int pair_h = 0, int dil = 1, float *ws = nullptr, size_t ws_floats = 0,
                                      const unsigned *pair_skip = nullptr, ImplicitLaunch *plan_only = nullptr)
{
    GemmParams p;
    p.A = wr; p.B = gyp; p.C = gx;
    p.M = C; p.K = Kf;
    p.n_img = H * Wp;
    p.N = B * p.n_img;
    const long long chan = phase != 0 ? 4LL * phase : (long long)Hp * Wp;  // elements per contracted channel of B
    p.lda = (long long)kh * kw * Kf; p.ldb = chan; p.ldc = (long long)H * W;
    p.sA = 0; p.sB = (long long)Kf * chan; p.sC = (long long)C * H * W;
    p.sAk = Kf; p.sBk = 0;
    p.kbatch = kh * kw; p.kb_per_split = p.kbatch; p.splits = 1; p.sCsplit = 0;
    p.alpha = 1.f; p.beta = 0.f;
    p.n_off = 0;
    p.conv_wp = Wp; p.conv_w = W; p.conv_kw = kw;
    p.conv_phase = phase;
    p.conv_dil = dil;
    p.conv_pair_w = pair_w; p.conv_pair_a = pair_a;
    p.conv_pair_grouped = pair_skip != nullptr;
    p.conv_pair_skip[0] = pair_skip ? pair_skip[0] : 0;
    p.conv_pair_skip[1] = pair_skip ? pair_skip[1] : 0;
    if (pair_w != 0) {
        p.ldc = (long long)pair_h * pair_w;
        p.sC = (long long)(C / 2) * pair_h * pair_w;
    }
    p.rows_taps = p.rows_kw = p.rows_wp = 0;
    p.rows_plane = p.rows_phase = 0;
    const long long out_floats = pair_w != 0 ? (long long)B * (C / 2) * pair_h * pair_w : (long long)B * C * H * W;
    const ImplicitPlan plan = implicit_plan(B, C, Kf, H, Wp, kh * kw, phase, pair_w,
                                            ws != nullptr && phase == 0 && pair_w == 0 && out_floats < 0x7fffffffLL &&
                                                ws_floats >= 2 * (size_t)out_floats);
    const int cfg = plan.cfg;
    AG_REQUIRE(!pair_skip || (cfg >= 13 && cfg <= 15) || cfg == 18, AG_ERR_INVALID_DIMS,
               "conv2d_transpose: rows grouped by parity need a tile whose waves hold 64 rows");
    p.kb_per_split = (int)cdiv(Kf / 32, plan.splits);
    p.splits = (int)cdiv(Kf / 32, p.kb_per_split);
    if ((size_t)p.splits * (size_t)out_floats > ws_floats) {  // (a forced split count the workspace cannot hold)
        p.splits = 1;
        p.kb_per_split = Kf / 32;
    }
    p.sCsplit = out_floats;
    if (p.splits > 1) p.C = ws;
    p.tiles_m = (int)cdiv(C, kCfgs[cfg].bm);
    p.tiles_n = (int)cdiv(p.N, kCfgs[cfg].bn);
    const long long blocks = (long long)p.tiles_m * p.tiles_n;
    AG_REQUIRE(blocks * p.splits <= kMaxGridX, AG_ERR_INVALID_DIMS, "conv2d_transpose: too many tiles (%lld)", blocks);
    p.total_blocks = (unsigned)(blocks * p.splits);
    // whole rounds of the persistent grid with the wide tile, then the remaining columns with a
    // narrower one (as for the folded GEMM over columns)
    int tail_cfg = -1;
    GemmParams tail = p;
    if (cfg == 14 && p.tiles_m == 1 && g_grid_scale <= 0 && p.splits == 1) {
        const long long G = direct_grid(num_cus());
        const long long rounds = blocks / G, rem = blocks % G;
        if (rounds >= 1 && rem > 0) {
            const int bn = kCfgs[cfg].bn;
            const long long main_cols = rounds * G * bn;
            double best = (double)rounds + 1.0 - 0.05;
            static const int narrow[] = {18, 13};  // 128 x 64, 128 x 128
            static const double eff[] = {0.85, 0.92};
            for (int t = 0; t < 2; ++t) {
                const int bnt = kCfgs[narrow[t]].bn;
                const long long items = cdiv(p.N - main_cols, bnt);
                const double cost = (double)rounds + (double)cdiv(items, G) * bnt / bn / eff[t];
                if (cost < best && p.n_img >= bnt) {
                    best = cost;
                    tail_cfg = narrow[t];
                }
            }
            if (tail_cfg >= 0) {
                tail.n_off = (int)main_cols;
                tail.tiles_n = (int)cdiv(p.N - main_cols, kCfgs[tail_cfg].bn);
                tail.total_blocks = (unsigned)tail.tiles_n;
                p.N = (int)main_cols;
                p.tiles_n = (int)(rounds * G);
                p.total_blocks = (unsigned)p.tiles_n;
            }
        }
    }
    if (plan_only != nullptr) {
        AG_REQUIRE(p.splits == 1, AG_ERR_INVALID_DIMS, "conv2d_transpose: a merged launch of a sliced product");
        plan_only->p = p;
        plan_only->tail = tail;
        plan_only->cfg = cfg;
        plan_only->tail_cfg = tail_cfg;
        return AG_OK;
    }
    launch_direct(st, cfg, true, false, p, num_cus(), g_grid_scale);
    if (ag_status_t s = check_launch("conv2d_transpose")) return s;
    if (tail_cfg >= 0) {
        launch_direct(st, tail_cfg, true, false, tail, num_cus(), g_grid_scale);
        return check_launch("conv2d_transpose");
    }
    if (p.splits > 1) {  // the partial results, slot after slot in ascending order of the channel groups
        launch_fold(st, ws, p.splits, out_floats, gx, 1, (int)out_floats, out_floats, 1.f, 0.f);
        return check_launch("conv2d_transpose");
    }
    return AG_OK;
}

static ImplicitPlan implicit_plan(int B, int C, int Kf, int H, int Wp, int taps, unsigned phase, int pair_w, bool may_split)
{
    const int n_img = H * Wp;
    const long long N = (long long)B * n_img;
    // 32 x 128 for up to 32 output rows; 64 x 128 for up to 64 (64 x 64 while that gives fewer than two blocks per
    // CU); else 128 x 256 (128 x 128 when an image has fewer than 256 columns) or 64 x 128, whichever needs less
    // time by rounds of the persistent grid times the cost of a tile: padding rows and the idle part of a last
    // round cost as much as real work (B = 128, 64 -> 192 channels, 28 x 28: 0.30 ms on 128 x 256 tiles -- 256
    // rows in 3.2 rounds -- against 0.21 ms on 64 x 128 ones)
    int cfg = C <= 32 ? kDirectCfg32 : kDirectCfg64;
    // Fewer 64-row tiles than fill the chip: each block takes a slice of the contraction instead of all of it (a
    // range of the Kf / 32 channel groups; partial results folded in a fixed order), as many slices as give about a
    // block per CU.  256 -> 256 channels, 14 x 14, dilation 2: 4 / 8 / 16 images 54 / 56 / 58 us whole, 23 / 33 / 55 us
    // sliced by 8 / 4 / 2; 8 images of 512 -> 512 channels at 7 x 7: 101 -> 33 us.  From about a block per CU on
    // slicing loses to whole contractions (32 images: 85 us whole on 64 x 128 tiles, 90 sliced by 2, 93 on 64 x 64 tiles).
    const int groups = Kf / 32;
    if (may_split && g_force_cfg < 0 && g_force_splits <= 0 && C > 32 && groups >= 2) {
        const long long G = direct_grid(num_cus());
        const int tile = C <= 64 ? kDirectCfg64Narrow : kDirectCfg64;
        const long long blocks = cdiv(C, 64) * cdiv(N, kCfgs[tile].bn);
        if (blocks * 5 < G * 3) {
            long long want = cdiv(G * 4, blocks * 5);
            if (want > 8) want = 8;
            if (want > groups) want = groups;
            const int per = (int)cdiv(groups, want);
            return ImplicitPlan{tile, (int)cdiv(groups, per)};
        }
    }
    if (C > 32 && C <= 64) {
        // (the stride-2 forms keep to tiles that cover at most two images)
        if (cdiv(N, 128) < 2 * direct_grid(num_cus()) && (n_img >= 64 || (phase == 0 && pair_w == 0))) cfg = kDirectCfg64Narrow;
    } else if (C > 64) {
        const long long G = direct_grid(num_cus());
        const int wide = n_img >= 256 ? 14 : 13;
        const long long wide_tiles = cdiv(C, 128) * cdiv(N, kCfgs[wide].bn);
        double wide_rounds = (double)cdiv(wide_tiles, G);
        if (wide == 14 && C <= 128 && wide_tiles > G && wide_tiles % G != 0)  // the narrow-tile tail launch below
            wide_rounds = (double)(wide_tiles / G) + 0.3;
        const double wide_cost = wide_rounds * 128.0 * kCfgs[wide].bn / (wide == 14 ? 1.0 : 0.9);
        const double small_cost = (double)cdiv(cdiv(C, 64) * cdiv(N, 128), 2 * G) * 2.0 * 64.0 * 128.0 / 0.95;
        cfg = wide_cost <= small_cost ? wide : kDirectCfg64;
        // a problem of less than a round of those: 64 x 64 tiles (32 x 256 -> 256 channels, 14 x 14: 0.100 against
        // 0.108 ms)
        // (only while the 64 x 128 tiles leave the chip well under a block per CU: with 224 of them on 256 CUs they
        // take 85 us where 448 tiles of 64 x 64 take 93)
        const double narrow_cost = (double)cdiv(cdiv(C, 64) * cdiv(N, 64), 2 * G) * 2.0 * 64.0 * 64.0 / 0.78;
        if (narrow_cost < 0.9 * (wide_cost <= small_cost ? wide_cost : small_cost) && cdiv(C, 64) * cdiv(N, 128) * 5 < G * 3)
            cfg = kDirectCfg64Narrow;
    }
    if (g_force_cfg >= kFirstDirectCfg && g_force_cfg < kNumCfgs && g_force_cfg != kDirectCfg32 && (pair_w == 0 && phase == 0 || kCfgs[g_force_cfg].bn <= n_img))
        cfg = g_force_cfg;  // test hook
    int splits = 1;
    if (g_force_splits > 0 && may_split) splits = g_force_splits < Kf / 32 ? g_force_splits : Kf / 32;  // test hook
    (void)taps;
    return ImplicitPlan{cfg, splits};
}

// Floats of workspace that gemm_conv_input_grad wants for the partial results of a split contraction (0: it
// will not split).
size_t gemm_conv_input_grad_ws_floats(int B, int C, int Kf, int H, int W, int Wp, int taps)
{
    const long long out = (long long)B * C * H * W;
    if (Kf < 64 || out >= (1LL << 26)) return 0;
#ifdef AG_TEST_HOOKS
    return (size_t)out * 8;  // room for forced split counts
#else
    const ImplicitPlan plan = implicit_plan(B, C, Kf, H, Wp, taps, 0, 0, true);
    return plan.splits > 1 ? (size_t)out * plan.splits : 0;
#endif
}

ag_status_t gemm_conv_input_grad(hipStream_t st, const float *wr, const float *gyp, float *gx, int B, int C,
                                 int Kf, int H, int W, int kh, int kw, int Hp, int Wp, int dil, float *ws, size_t ws_floats)
{
    return conv_implicit_gemm(st, wr, gyp, gx, B, C, Kf, H, W, kh, kw, Hp, Wp, 0, 0, 0, 0, dil, ws, ws_floats);
}

ag_status_t gemm_conv_input_grad_pair(hipStream_t st, const float *wr, const float *gyp, float *gx, int B, int C, int Kf, int Ha,
                                      int Wb, int kh, int kw, int Hp, int Wp, int a, int Hout, int Wout, const unsigned *skip)
{
    return conv_implicit_gemm(st, wr, gyp, gx, B, 2 * C, Kf, Ha, Wb, kh, kw, Hp, Wp, 0, Wout, a, Hout, 1, nullptr, 0, skip);
}

// Both row parities of the grouped pair form.  Where the two products run on the same tiles they share their launches
// (launch_direct's `second`): a CU that has finished its tiles of parity 0 goes on with parity 1 instead of waiting for
// the other CUs, and the two narrow tails fill one round together.
ag_status_t gemm_conv_input_grad_pair_both(hipStream_t st, const float *const wr[2], const float *const gyp[2], float *gx, int B,
                                           int C, int Kf, const int Ha[2], int Wb, const int kh[2], int kw, int Hp, int Wp,
                                           int Hout, int Wout, const unsigned *const skip[2])
{
    ImplicitLaunch L[2];
    for (int a = 0; a < 2; ++a)
        if (ag_status_t s = conv_implicit_gemm(st, wr[a], gyp[a], gx, B, 2 * C, Kf, Ha[a], Wb, kh[a], kw, Hp, Wp, 0, Wout, a, Hout,
                                               1, nullptr, 0, skip[a], &L[a]))
            return s;
    const bool merge = L[0].cfg == L[1].cfg && L[0].tail_cfg == L[1].tail_cfg && g_grid_scale <= 0 &&
                       ((L[0].cfg >= 13 && L[0].cfg <= 15) || L[0].cfg == 18) && (L[0].tail_cfg < 0 || L[0].tail_cfg == 13 || L[0].tail_cfg == 18);
    if (merge) {
        launch_direct(st, L[0].cfg, true, false, L[0].p, num_cus(), g_grid_scale, &L[1].p);
        if (ag_status_t s = check_launch("conv2d_transpose")) return s;
        if (L[0].tail_cfg >= 0) {
            launch_direct(st, L[0].tail_cfg, true, false, L[0].tail, num_cus(), g_grid_scale, &L[1].tail);
            return check_launch("conv2d_transpose");
        }
        return AG_OK;
    }
    for (int a = 0; a < 2; ++a) {
        launch_direct(st, L[a].cfg, true, false, L[a].p, num_cus(), g_grid_scale);
        if (ag_status_t s = check_launch("conv2d_transpose")) return s;
        if (L[a].tail_cfg >= 0) {
            launch_direct(st, L[a].tail_cfg, true, false, L[a].tail, num_cus(), g_grid_scale);
            if (ag_status_t s = check_launch("conv2d_transpose")) return s;
        }
    }
    return AG_OK;
}

// The tiles whose waves hold 64 rows (two 32-row blocks, one per parity): 128 x 128, 128 x 256, 256 x 128, 128 x 64.
bool gemm_conv_input_grad_pair_grouped(int B, int C, int Kf, int Ha, int Wp, int taps)
{
    if (g_force_cfg >= 0) return false;  // (a forced tile may be one of the others)
    const int cfg = implicit_plan(B, 2 * C, Kf, Ha, Wp, taps, 0, 1, false).cfg;
    return (cfg >= 13 && cfg <= 15) || cfg == 18;
}

ag_status_t gemm_conv_fwd_stride2(hipStream_t st, const float *wf, const float *xph, float *y, int B, int K, int C,
                                  int OH, int OW, int kh, int kw, int Hpp, int Wpp)
{
    return conv_implicit_gemm(st, wf, xph, y, B, K, C, OH, OW, kh, kw, Hpp, Wpp, (unsigned)(Hpp * Wpp));
}

// Tile of the implicit filter gradient (both operands k-contiguous): 128 x 192; for up to 64 or 32 filters tiles of
// that many rows, since the padding rows of a taller tile cost as much as real ones (B = 256, 32 -> 64 channels,
// 56 x 56: 0.61 ms on 128-row tiles, 0.36 ms on 64-row ones).
static int conv_filter_grad_cfg(int Kf, long long cols)
{
    if (g_force_cfg >= kFirstDirectCfg && g_force_cfg < kNumCfgs) return g_force_cfg;  // test hook
    if (Kf <= 32) return kDirectCfg32;
    if (Kf <= 64) return cols >= 512 ? kDirectCfg64 : kDirectCfg64Narrow;
    // 192 x 128 where that pads less (160 or 192 filters: 0.90 against 1.21 ms at B = 64, 160 -> 160, 56 x 56)
    const double tall = (double)(cdiv(Kf, 192) * 192) * (double)(cdiv(cols, 128) * 128) / 0.95;
    const double wide = (double)(cdiv(Kf, 128) * 128) * (double)(cdiv(cols, 192) * 192);
    return tall < wide ? 16 : 17;
}

static int conv_filter_grad_splits(int B, int Kf, int C, int taps, int kq)
{
    (void)kq;
    // as many splits as give the chip a few rounds of tiles; every split sums whole images
    const int cfg = conv_filter_grad_cfg(Kf, (long long)C * taps);
    const long long tiles = cdiv(Kf, kCfgs[cfg].bm) * cdiv((long long)C * taps, kCfgs[cfg].bn);
    long long want = cdiv(kCfgs[cfg].bm <= 64 ? 1024 : 4096, tiles);
    if (g_force_splits > 0) want = g_force_splits;  // test hook
    if (want > B) want = B;
    const long long per = cdiv(B, want);
    return (int)cdiv(B, per);
}

// A block that sums one whole image is as fine as the splits get, and it takes a fixed time (0.28 ms for a 56 x 56
// plane on a 128 x 192 tile) however few of them there are: below about a hundred images the chip would be part
// empty for that long.  Small batches therefore also cut the flattened plane into equal chunks of positions, which
// the kernel sees as a batch of independent products (origins a chunk apart), each with partial sums of its own;
// the fold adds them all in a fixed order.  Returns the number of chunks (a divisor of the plane's k tiles).
static int conv_filter_grad_chunks(int B, int Kf, int C, int taps, int kq)
{
    if (kq < 512 || kq % 32 != 0) return 1;
    const int cfg = conv_filter_grad_cfg(Kf, (long long)C * taps);
    const long long tiles = cdiv(Kf, kCfgs[cfg].bm) * cdiv((long long)C * taps, kCfgs[cfg].bn);
    const long long blocks = tiles * conv_filter_grad_splits(B, Kf, C, taps, kq);
    if (blocks >= 768) return 1;
    long long want = cdiv(1024, blocks);
    const int kt = kq / 32;
    if (want > kt / 8) want = kt / 8;  // at least eight k tiles per chunk
    for (long long c = want; c >= 2; --c)
        if (kt % c == 0) return (int)c;
    return 1;
}

size_t gemm_conv_filter_grad_workspace(int B, int Kf, int C, int taps, int kq)
{
    const long long partials = (long long)conv_filter_grad_splits(B, Kf, C, taps, kq) * conv_filter_grad_chunks(B, Kf, C, taps, kq);
    return partials > 1 ? sizeof(float) * (size_t)partials * Kf * C * taps : 16;
}

// a_plane / b_plane: elements per row of A (one filter's gradient plane) and per channel of B; phase != 0: B is
// split into four phase planes per channel (stride 2).
static ag_status_t conv_filter_grad_gemm(hipStream_t st, const float *a, const float *xp, float *gw, void *ws, size_t ws_bytes,
                                         int B, int Kf, int C, int kh, int kw, int Wp, int kq, long long a_plane,
                                         long long b_plane, unsigned phase, int dil = 1)
{
    const int taps = kh * kw;
    GemmParams p;
    p.A = a;
    p.B = xp;
    p.M = Kf; p.N = C * taps; p.K = kq;
    p.lda = a_plane; p.ldb = b_plane; p.ldc = p.N;
    p.sA = p.sB = p.sC = 0;
    p.sAk = (long long)Kf * a_plane; p.sBk = (long long)C * b_plane;
    p.kbatch = B;
    p.splits = conv_filter_grad_splits(B, Kf, C, taps, kq);
    p.kb_per_split = (int)cdiv(B, p.splits);
    p.splits = (int)cdiv(B, p.kb_per_split);
    p.sCsplit = (long long)p.M * p.N;
    p.alpha = 1.f; p.beta = 0.f;
    p.n_img = 0; p.n_off = 0;
    p.conv_wp = p.conv_w = p.conv_kw = 0;
    p.conv_pair_w = p.conv_pair_a = 0;
    p.conv_pair_grouped = 0;
    p.conv_pair_skip[0] = p.conv_pair_skip[1] = 0;
    p.conv_phase = 0;
    p.conv_dil = dil;
    p.rows_taps = taps; p.rows_kw = kw; p.rows_wp = Wp; p.rows_plane = (unsigned)b_plane; p.rows_phase = phase;
    p.C = gw;
    // (the stride-2 form keeps whole planes: its workspace is sized without knowing kq)
    const int chunks = phase == 0 ? conv_filter_grad_chunks(B, Kf, C, taps, kq) : 1;
    const long long partials = (long long)p.splits * chunks;
    // chunk z of every plane is "batch" z of the product: origins kq / chunks positions apart, partial sums in the
    // slots z * splits .. z * splits + splits - 1
    p.K = kq / chunks;
    p.sA = p.sB = p.K;
    p.sC = (long long)p.splits * p.sCsplit;
    if (partials > 1) {
        const size_t need = sizeof(float) * (size_t)partials * p.M * p.N;
        AG_REQUIRE(ws && ws_bytes >= need, AG_ERR_INVALID_DIMS, "conv2d_filter_grad: workspace of %zu bytes needed, %zu given",
                   need, ws_bytes);
    }
    const int cfg = conv_filter_grad_cfg(Kf, (long long)C * taps);
    p.tiles_m = (int)cdiv(p.M, kCfgs[cfg].bm);
    p.tiles_n = (int)cdiv(p.N, kCfgs[cfg].bn);
    p.total_blocks = (unsigned)((long long)p.tiles_m * p.tiles_n * partials);
    if (partials > 1) p.C = static_cast<float *>(ws);
    launch_direct(st, cfg, true, true, p, num_cus(), g_grid_scale);
    if (ag_status_t e = check_launch("conv2d_filter_grad")) return e;
    if (partials > 1) {
        launch_fold(st, static_cast<const float *>(ws), (int)partials, p.sCsplit, gw, p.M, p.N, (long long)p.N, 1.f, 0.f);
        return check_launch("conv2d_filter_grad");
    }
    return AG_OK;
}

ag_status_t gemm_conv_filter_grad(hipStream_t st, const float *gyp, const float *xp, float *gw, void *ws, size_t ws_bytes,
                                  int B, int Kf, int C, int kh, int kw, int border, int Hp_gy, int Hp_x, int Wp, int kq, int dil)
{
    // positions are counted from the first gradient value, `border` rows and elements into a plane of gyp
    return conv_filter_grad_gemm(st, gyp + ((long long)border * Wp + border), xp, gw, ws, ws_bytes, B, Kf, C, kh, kw, Wp, kq,
                                 (long long)Hp_gy * Wp, (long long)Hp_x * Wp, 0, dil);
}

size_t gemm_conv_filter_grad_stride2_workspace(int B, int Kf, int C, int taps)
{
    return gemm_conv_filter_grad_workspace(B, Kf, C, taps, 0);
}

ag_status_t gemm_conv_filter_grad_stride2(hipStream_t st, const float *gyq, const float *xph, float *gw, void *ws,
                                          size_t ws_bytes, int B, int Kf, int C, int kh, int kw, int Hq, int Hpp, int Wpp, int kq)
{
    const long long pp = (long long)Hpp * Wpp;
    return conv_filter_grad_gemm(st, gyq, xph, gw, ws, ws_bytes, B, Kf, C, kh, kw, Wpp, kq, (long long)Hq * Wpp, 4 * pp,
                                 (unsigned)pp);
}

// Number of splits for an accumulated-batch GEMM: enough blocks for a few waves over the chip.
static int choose_splits(int M, int N, int K, int kbatch)
{
    if (g_force_splits > 0) return g_force_splits < kbatch ? g_force_splits : kbatch;
    // tile choice as if every image were a block; the alignment of the operands is not known here
    const int cfg = choose_cfg(M, N, K, kbatch, true, K % 32 == 0);
    const long long tiles = cdiv(M, kCfgs[cfg].bm) * cdiv(N, kCfgs[cfg].bn);
    long long want = cdiv(4096, tiles);
    if (want > kbatch) want = kbatch;
    if (want < 1) want = 1;
    // make the splits even
    const long long per = cdiv(kbatch, want);
    return (int)cdiv(kbatch, per);
}

// A single product with few output tiles and a long contraction is cut into `s` slices of the
// contraction that are summed like the images of an accumulated-batch GEMM, so that more than a
// handful of blocks work on it.  Returns s (1 = no split); K / s is a multiple of 4.
static int matmul_slices(int M, int N, int K)
{
    const long long tiles = cdiv(M, 64) * cdiv(N, 64);
    if (tiles >= 64 || K < 512) return 1;
    long long want = cdiv(256, tiles);
    if (want > K / 64) want = K / 64;
    for (long long s = want; s >= 2; --s)
        if (K % s == 0 && (K / s) % 4 == 0) return (int)s;
    return 1;
}

}  // namespace ag

using namespace ag;

#ifdef AG_TEST_HOOKS
// Test hooks (ag_test_hooks.h; not part of the operator surface and not in the shipped library).  Each sets a
// thread-local override that later calls made by the same thread observe.
extern "C" void ag_test_gemm_force_config(int cfg) { g_force_cfg = cfg; }
extern "C" void ag_test_gemm_force_splits(int splits) { g_force_splits = splits; }
extern "C" void ag_test_gemm_force_grid(int blocks_per_cu) { g_grid_scale = blocks_per_cu; }
#endif

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
    if (M <= 0 || N <= 0 || batch <= 0) return 16;
    const int splits = choose_splits(M, N, K, batch);
    // a contraction with a K tail runs as two passes that keep their partial sums side by side
    const size_t passes = (K % 32 != 0 && K >= 256) ? 2 : 1;
    return splits > 1 ? sizeof(float) * passes * (size_t)splits * M * N : 16;
}

extern "C" ag_status_t ag_gemm_batchsum_f32(ag_stream_t stream, int transA, int transB, int M, int N, int K,
                                            float alpha, const float *A, int lda, long long strideA,
                                            const float *B, int ldb, long long strideB, float beta, float *C,
                                            int ldc, int batch, void *ws, size_t ws_bytes)
{
    GemmCall c{transA, transB, M, N, K, alpha, beta, A, lda, 0, strideA, B, ldb, 0, strideB, C, ldc, 0, 1, batch};
    const int splits = (M > 0 && N > 0 && batch > 0) ? choose_splits(M, N, K, batch) : 1;
    return run_gemm(as_stream(stream), "gemm_batchsum", c, ws, ws_bytes, splits);
}

extern "C" size_t ag_matmul_f32_workspace(int M, int N, int K)
{
    if (M <= 0 || N <= 0 || K <= 0) return 16;
    const int s = matmul_slices(M, N, K);
    return s > 1 ? ag_gemm_batchsum_f32_workspace(M, N, K / s, s) : 16;
}

extern "C" ag_status_t ag_matmul_f32(ag_stream_t stream, int transA, int transB, int M, int N, int K, const float *A,
                                     int lda, const float *B, int ldb, float *C, int ldc, void *ws, size_t ws_bytes)
{
    const int s = (M > 0 && N > 0 && K > 0) ? matmul_slices(M, N, K) : 1;
    if (s <= 1) return ag_gemm_f32(stream, transA, transB, M, N, K, 1.f, A, lda, 0, B, ldb, 0, 0.f, C, ldc, 0, 1);
    const int Kc = K / s;
    // slice i of the contraction: columns of op(A), rows of op(B)
    const long long strideA = transA ? (long long)Kc * lda : Kc;
    const long long strideB = transB ? Kc : (long long)Kc * ldb;
    return ag_gemm_batchsum_f32(stream, transA, transB, M, N, Kc, 1.f, A, lda, strideA, B, ldb, strideB, 0.f, C, ldc, s, ws,
                                ws_bytes);
}

// ---------------------------------------------------------------------------------------------
// ag_matmul_f32 for callers that cannot allocate (code under HIP graph capture, serving loops,
// harnesses that forbid hipMalloc): the partial sums of a sliced contraction go to a fixed device
// array of this library instead of a caller workspace.  Every GPU the library runs on holds its
// own copy of the array until the process ends; its address on a device is looked up once, with
// that device current, and only that address (never the array's name, which is a host-side
// stand-in) is handed to kernels.  Calls that overlap on one GPU share the array and race.
// ---------------------------------------------------------------------------------------------
namespace ag {

constexpr size_t kStaticScratchBytes = 4u << 20;  // 4 MiB per GPU
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void *g_scratch_ptr[kMaxDevices] = {};  // per device, guarded by g_scratch_mutex

static ag_status_t static_scratch(void **out)
{
    int dev = -1;
    if (ag_status_t s = check_hip(hipGetDevice(&dev), "matmul (static scratch): hipGetDevice")) return s;
    AG_REQUIRE(dev >= 0 && dev < kMaxDevices, AG_ERR_INVALID_DIMS, "matmul (static scratch): device %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        if (ag_status_t s = check_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)),
                                      "matmul (static scratch): hipGetSymbolAddress"))
            return s;
        AG_REQUIRE(ptr, AG_ERR_INVALID_DIMS, "matmul (static scratch): null symbol address");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return AG_OK;
}

}  // namespace ag

extern "C" size_t ag_matmul_f32_static_scratch_bytes(void) { return ag::kStaticScratchBytes; }

extern "C" ag_status_t ag_matmul_f32_noalloc(ag_stream_t stream, int transA, int transB, int M, int N, int K,
                                             const float *A, int lda, const float *B, int ldb, float *C, int ldc)
{
    const size_t need = ag_matmul_f32_workspace(M, N, K);
    if (need <= 16)  // not sliced: no scratch involved
        return ag_matmul_f32(stream, transA, transB, M, N, K, A, lda, B, ldb, C, ldc, nullptr, 0);
    AG_REQUIRE(need <= ag::kStaticScratchBytes, AG_ERR_INVALID_DIMS,
               "matmul (no allocation): %d x %d x %d needs %zu bytes of scratch, the fixed array holds %zu; "
               "use ag_matmul_f32 with a caller workspace",
               M, N, K, need, ag::kStaticScratchBytes);
    void *ws = nullptr;
    if (ag_status_t s = ag::static_scratch(&ws)) return s;
    // every slot the fold reads is written by this call's GEMM first: nothing needs clearing
    return ag_matmul_f32(stream, transA, transB, M, N, K, A, lda, B, ldb, C, ldc, ws, need);
}
