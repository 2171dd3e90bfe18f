// fp32 GEMM on the matrix cores with operand tiles loaded from global memory straight into LDS.

#include <type_traits>

#include "gemm_shared.h"

namespace ag {

// ---------------------------------------------------------------------------------------------
// Direct-to-LDS variant.  gfx950 can load 16 bytes per lane from global memory straight into LDS
// (global_load_lds_dwordx4): lane l of a wave deposits its 16 bytes at LDS base + 16*l, whatever
// global address it fetched.  Operand tiles therefore never pass through registers; the layout
// in LDS is made conflict-free by choosing WHICH 16-byte chunk each lane fetches (an XOR swizzle
// on the global side) instead of by padding.  BK = 32.
//
//   k-contiguous operand (rows x 32 k):  row r, chunk c (4 k) lives at chunk position
//       r*8 + (c ^ f(r)),  f(r) = (r & 7) ^ ((r >> 3) & 1);
//     a lane reads four consecutive k of its row with one 128-bit LDS read.
//   m/n-contiguous operand (32 k x rows): element (k, n) lives at k*rows + (n ^ (32 * ((k>>2)&1)));
//     a lane reads one k of its column per MFMA step with 32-bit LDS reads (the two half-waves
//     read k and k+4, which the swizzle puts 128 bytes apart).
//
// The ring has STAGES slots; loads run STAGES-1 k tiles ahead of the MFMAs.  Each k tile has one
// barrier, in its middle: before it a wave waits (vmcnt) until the NEXT tile's loads have
// landed, after it the slot of the PREVIOUS tile is free for the loads issued next.  The loads
// and the wait are inline assembly because the compiler would otherwise put a full vmcnt(0)
// in front of every LDS read that follows an LDS-writing load; vmcnt counts loads and stores in
// issue order, so "at most n outstanding" identifies which tiles have landed.
// Requirements (checked on the host, else the register-staged kernel above runs): K % 32 == 0,
// 16-byte aligned operands, leading dimensions and batch strides multiples of 4, and for an
// m/n-contiguous operand an extent that is a multiple of 4.
// ---------------------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) float lds_float_t;

// One wave-level 1 KiB load: lane l fetches 16 bytes at base + byte_off and they land at LDS byte
// address lds_wave_base + LDS_IMM + 16*l.  (m0 carries the LDS address; a write to m0 needs one
// wait state before the load that uses it.)
template <int LDS_IMM>
__device__ inline void dma16(const float *base, unsigned byte_off, unsigned lds_wave_base)
{
    // (the base is wave-uniform; naming its halves as first-lane values keeps it in scalar registers for the
    // assembly below whatever the compiler did with the pointer arithmetic before -- free when it is there already)
    const unsigned long long bits = reinterpret_cast<unsigned long long>(base);
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)bits);
    const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(bits >> 32));
    const float *sbase = reinterpret_cast<const float *>(((unsigned long long)hi << 32) | lo);
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_wave_base), "v"(byte_off), "s"(sbase), "n"(LDS_IMM)
                 : "m0", "scc");
}

template <int N>
__device__ inline void wait_loads_then_barrier()
{
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "n"(N) : "memory");
}

// Swizzle of a k-contiguous tile: which 16-byte chunk position of row r holds chunk c.
template <int BK>
__device__ inline int kc_swizzle(int r)
{
    return BK == 32 ? ((r & 7) ^ ((r >> 3) & 1)) : (((r >> 1) ^ (r >> 3)) & 3);
}

template <bool KC, int ROWS, int BK, int NW>
struct DirectTile {
    static constexpr int CPR = KC ? BK / 4 : ROWS / 4;  // 16-byte chunks per LDS row
    static constexpr int INSTR = ROWS * BK / 4 / 64;    // wave-level 1 KiB loads per tile
    static constexpr int PER_WAVE = INSTR / NW;
    static_assert(INSTR % NW == 0 && PER_WAVE >= 1, "tile does not divide over the waves");
    static_assert(KC || ROWS % 64 == 0, "m/n-contiguous tiles are swizzled in 64-element groups");

    unsigned off[PER_WAVE];  // byte offset of this lane's chunk from the k-tile origin

    __device__ inline void init(int ld, int row0, int rows, int wave, int lane)
    {
#pragma unroll
        for (int i = 0; i < PER_WAVE; ++i) {
            const int pos = (i * NW + wave) * 64 + lane;  // chunk position in the LDS tile
            if (KC) {
                const int r = pos / CPR, c = (pos % CPR) ^ kc_swizzle<BK>(r);
                const int row = min(row0 + r, rows - 1);
                off[i] = (unsigned)(row * ld + c * 4) * 4u;
            } else {
                const int k = pos / CPR, cn = (pos % CPR) ^ (((k >> 2) & 1) * 8);
                const int n = min(row0 + cn * 4, rows - 4);
                off[i] = (unsigned)(k * ld + n) * 4u;
            }
        }
    }
    // k-contiguous rows that are (channel, tap) pairs of a zero-bordered input (implicit filter
    // gradient): row n starts (n / taps) * plane + (ky * wp + kx) * dil elements after the origin.
    // `phase` != 0 (stride 2): the input is split into four phase planes of `phase` elements each and
    // tap (ky, kx) reads phase (ky&1, kx&1) shifted by (ky>>1) rows and (kx>>1) elements.
    __device__ inline void init_conv_rows(int row0, int rows, int taps, int kw, int wp, unsigned plane, unsigned phase,
                                          int dil, int wave, int lane)
    {
#pragma unroll
        for (int i = 0; i < PER_WAVE; ++i) {
            const int pos = (i * NW + wave) * 64 + lane;
            const int r = pos / CPR, c = (pos % CPR) ^ kc_swizzle<BK>(r);
            const int row = min(row0 + r, rows - 1);
            const int ch = row / taps, tap = row - ch * taps;
            const int ky = tap / kw, kx = tap - ky * kw;
            const unsigned shift = phase != 0 ? (unsigned)((ky & 1) * 2 + (kx & 1)) * phase + (unsigned)((ky >> 1) * wp + (kx >> 1))
                                              : (unsigned)((ky * wp + kx) * dil);
            off[i] = ((unsigned)ch * plane + shift + (unsigned)(c * 4)) * 4u;
        }
    }
    // Folded batch (m/n-contiguous operand only): the tile starts at column r0 of one batch and
    // may run on into the next one, `next` elements further (0 when there is no next batch: those
    // columns are clamped like any column beyond the operand).
    __device__ inline void init_folded(int ld, int r0, int n_img, unsigned next, int wave, int lane)
    {
#pragma unroll
        for (int i = 0; i < PER_WAVE; ++i) {
            const int pos = (i * NW + wave) * 64 + lane;
            const int k = pos / CPR, cn = (pos % CPR) ^ (((k >> 2) & 1) * 8);
            int n = r0 + cn * 4;
            unsigned extra = 0;
            if (n >= n_img) {
                if (next != 0) {
                    n -= n_img;
                    extra = next;
                } else {
                    n = n_img - 4;
                }
            }
            off[i] = ((unsigned)(k * ld + n) + extra) * 4u;
        }
    }
    // The same for batches narrower than a tile (the 7 x 7 planes of a late convolution layer): a tile may run over
    // any number of them, `left` batches remain from the one it starts in (that one included).
    __device__ inline void init_folded_many(int ld, int r0, int n_img, int left, unsigned next, int wave, int lane)
    {
#pragma unroll
        for (int i = 0; i < PER_WAVE; ++i) {
            const int pos = (i * NW + wave) * 64 + lane;
            const int k = pos / CPR, cn = (pos % CPR) ^ (((k >> 2) & 1) * 8);
            int n = r0 + cn * 4;
            int q = n / n_img;
            n -= q * n_img;
            if (q >= left) {  // beyond the operand: clamped
                q = left - 1;
                n = n_img - 4;
            }
            off[i] = ((unsigned)(k * ld + n) + (unsigned)q * next) * 4u;
        }
    }
    __device__ static inline long long k_step(int ld) { return KC ? BK : (long long)BK * ld; }

    // Load number `i` (a constant after unrolling) of this wave.
    __device__ inline void issue_one(int i, const float *origin, unsigned lds_wave_base) const
    {
        if (i == 0 && 0 < PER_WAVE) dma16<0 * NW * 1024>(origin, off[0], lds_wave_base);
        if (i == 1 && 1 < PER_WAVE) dma16<1 * NW * 1024>(origin, off[1 < PER_WAVE ? 1 : 0], lds_wave_base);
        if (i == 2 && 2 < PER_WAVE) dma16<2 * NW * 1024>(origin, off[2 < PER_WAVE ? 2 : 0], lds_wave_base);
        if (i == 3 && 3 < PER_WAVE) dma16<3 * NW * 1024>(origin, off[3 < PER_WAVE ? 3 : 0], lds_wave_base);
        if (i == 4 && 4 < PER_WAVE) dma16<4 * NW * 1024>(origin, off[4 < PER_WAVE ? 4 : 0], lds_wave_base);
        if (i == 5 && 5 < PER_WAVE) dma16<5 * NW * 1024>(origin, off[5 < PER_WAVE ? 5 : 0], lds_wave_base);
        if (i == 6 && 6 < PER_WAVE) dma16<6 * NW * 1024>(origin, off[6 < PER_WAVE ? 6 : 0], lds_wave_base);
        if (i == 7 && 7 < PER_WAVE) dma16<7 * NW * 1024>(origin, off[7 < PER_WAVE ? 7 : 0], lds_wave_base);
    }

    // lds_wave_base: LDS byte address of the tile + 1024 * wave.
    template <int I0, int I1>
    __device__ inline void issue(const float *origin, unsigned lds_wave_base) const
    {
        // the LDS immediate must be a constant expression: unrolled by hand
        if (I0 <= 0 && 0 < I1 && 0 < PER_WAVE) dma16<0 * NW * 1024>(origin, off[0], lds_wave_base);
        if (I0 <= 1 && 1 < I1 && 1 < PER_WAVE) dma16<1 * NW * 1024>(origin, off[1 < PER_WAVE ? 1 : 0], lds_wave_base);
        if (I0 <= 2 && 2 < I1 && 2 < PER_WAVE) dma16<2 * NW * 1024>(origin, off[2 < PER_WAVE ? 2 : 0], lds_wave_base);
        if (I0 <= 3 && 3 < I1 && 3 < PER_WAVE) dma16<3 * NW * 1024>(origin, off[3 < PER_WAVE ? 3 : 0], lds_wave_base);
        if (I0 <= 4 && 4 < I1 && 4 < PER_WAVE) dma16<4 * NW * 1024>(origin, off[4 < PER_WAVE ? 4 : 0], lds_wave_base);
        if (I0 <= 5 && 5 < I1 && 5 < PER_WAVE) dma16<5 * NW * 1024>(origin, off[5 < PER_WAVE ? 5 : 0], lds_wave_base);
        if (I0 <= 6 && 6 < I1 && 6 < PER_WAVE) dma16<6 * NW * 1024>(origin, off[6 < PER_WAVE ? 6 : 0], lds_wave_base);
        if (I0 <= 7 && 7 < I1 && 7 < PER_WAVE) dma16<7 * NW * 1024>(origin, off[7 < PER_WAVE ? 7 : 0], lds_wave_base);
        static_assert(PER_WAVE <= 8, "at most eight loads per wave and operand");
    }
};

// CONV: how the k loop walks its operands, a template parameter because the scalar work between two k tiles sits on
// the critical path of the loads.  With the dilation as a kernel argument (a variable tap step instead of the
// constant 1) the undilated forward product of the headline step took 0.930 instead of 0.916 ms; with the tests
// "is this a convolution / a phase walk" decided at compile time it takes 0.905 ms, the input gradient 0.937
// instead of 0.964, the filter gradient 0.868 instead of 0.906 and the 4096^3 NT / TN products 0.965 / 0.971
// instead of 0.994 / 0.996 ms; the stride-2 forward over phase planes 0.291 instead of 0.300 ms.
// `bid` / `gdim`: this block's index and the number of blocks that share the product's work items (the whole grid,
// or one of the two parts of a grid that carries two products).
template <int BM, int BN, int BK, int WM, int WN, int STAGES, bool KA, bool KB, int CONV>
__device__ __forceinline__ void gemm_dl_body(const GemmParams &p, const unsigned bid, const unsigned gdim)
{
    // CONV 1 / 2: the tap walk of the implicit convolution (conv_wp != 0, no phase planes), without / with
    // dilation; 3: an ordinary product; 4: the stride-2 forward, whose taps walk the four phase planes; 5: the walk
    // of 1 for the pair form of the stride-2 input gradient with its rows grouped by parity, which leaves out the
    // matrix instructions of a parity at the taps it does not have
    static_assert(CONV >= 1 && CONV <= 5, "walk of the k loop");
    constexpr bool grouped = CONV == 5;
    static_assert(!grouped || WM == 64, "one 32-row block per parity and wave");
    constexpr bool shifts = CONV == 1 || CONV == 2 || CONV == 5;  // taps as shifts within one plane
    constexpr bool phases = CONV == 4;
    constexpr bool taps = shifts || phases;
    const int conv_dil = CONV == 2 ? p.conv_dil : 1;
    static_assert(STAGES >= 3 && STAGES <= 8, "ring of three to eight tiles");
    static_assert(BK == 16 || BK == 32, "k tile");
    constexpr int KK = BK / 8;  // groups of four MFMA k steps per tile
    constexpr int WAVES_N = BN / WN;
    constexpr int NW = (BM / WM) * (BN / WN);
    constexpr int MI = WM / 32, NI = WN / 32;
    constexpr int TILE = (BM + BN) * BK;  // floats per ring slot
    using LoadA = DirectTile<KA, BM, BK, NW>;
    using LoadB = DirectTile<KB, BN, BK, NW>;
    constexpr int L = LoadA::PER_WAVE + LoadB::PER_WAVE;  // loads per wave per k tile
    constexpr int STORES = MI * NI * 16;                  // epilogue stores per wave
    constexpr int STEADY = (STAGES - 3) * L;              // loads that may stay in flight at a tile's barrier
    constexpr int AFTER_EPILOGUE = STEADY + STORES > 63 ? 63 : STEADY + STORES;
    static_assert((STAGES - 2) * L <= 63, "vmcnt range");

    __shared__ __attribute__((aligned(1024))) float lds[STAGES * TILE];
    const unsigned lds_base = (unsigned)(size_t)(lds_float_t *)lds;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l31 = lane & 31, half = lane >> 5;
    const unsigned lds_wave = lds_base + (unsigned)wave * 1024u;

    const unsigned total = p.total_blocks;
    const unsigned tiles = (unsigned)(p.tiles_m * p.tiles_n);
    const int kt_per = p.K / BK;
    const int lda = (int)p.lda, ldb = (int)p.ldb;
    // pointer steps of the fetch stream: to the next k tile, and from the last k tile of one
    // accumulated batch to the first of the next
    const long long step_a = LoadA::k_step(lda), step_b = LoadB::k_step(ldb);
    const long long wrap_a = p.sAk - (kt_per - 1) * step_a, wrap_b = p.sBk - (kt_per - 1) * step_b;

    struct Item {
        int m0, n0, bz, sp, kb0, nt;
        int r0;  // folded batch: n0 = bz * n_img + r0
    };
    // Item w has the logical position xcd_remap(w) = (z * tiles_n + tn) * tiles_m + tm.  The block
    // walks items blockIdx.x, blockIdx.x + gridDim.x, ...; with the grid a multiple of the XCD
    // count (the host sees to it) the logical position advances by gridDim.x / 8 every time, so
    // the (tm, tn, z) digits are stepped with a few scalar adds instead of being divided out
    // again for every item.
    struct Cursor {
        int tm, tn, z;
    };
    Cursor step, first;
    {
        const unsigned stride = gdim / kXcds;
        step.tm = (int)(stride % (unsigned)p.tiles_m);
        step.tn = (int)(stride / (unsigned)p.tiles_m % (unsigned)p.tiles_n);
        step.z = (int)(stride / tiles);
        unsigned g = xcd_remap(bid, total);
        first.tm = (int)(g % (unsigned)p.tiles_m);
        g /= (unsigned)p.tiles_m;
        first.tn = (int)(g % (unsigned)p.tiles_n);
        first.z = (int)(g / (unsigned)p.tiles_n);
    }
    auto cursor_next = [&](Cursor &c) {
        c.tm += step.tm;
        const int carry_m = c.tm >= p.tiles_m;
        c.tm -= carry_m ? p.tiles_m : 0;
        c.tn += step.tn + carry_m;
        const int carry_n = c.tn >= p.tiles_n;
        c.tn -= carry_n ? p.tiles_n : 0;
        c.z += step.z + carry_n;
    };
    auto item_of = [&](const Cursor &c) {
        Item it;
        it.m0 = c.tm * BM;
        it.n0 = p.n_off + c.tn * BN;
        it.r0 = 0;
        if (p.n_img != 0) {
            it.bz = it.n0 / p.n_img;
            it.r0 = it.n0 - it.bz * p.n_img;
            it.sp = c.z;  // (only the tap walks are ever split: groups of 32 contracted channels)
        } else if (p.splits == 1) {
            it.bz = c.z;
            it.sp = 0;
        } else {
            it.bz = c.z / p.splits;
            it.sp = c.z % p.splits;
        }
        it.kb0 = it.sp * p.kb_per_split;
        if (taps) {
            // A tap walk visits every tap for one group of 32 contracted channels, then the next group: a split owns
            // kb_per_split consecutive groups (all of them when the walk is not split).
            it.nt = (min(kt_per, it.kb0 + p.kb_per_split) - it.kb0) * p.kbatch;
        } else {
            it.nt = (min(p.kbatch, it.kb0 + p.kb_per_split) - it.kb0) * kt_per;
        }
        return it;
    };

    // ---- fetch stream ----
    unsigned fw = bid;
    bool f_valid = fw < total;
    if (!f_valid) return;
    LoadA ldr_a;
    LoadB ldr_b;
    const float *pa = nullptr, *pb = nullptr;  // origin of the next k tile to fetch
    const float *pb_group = nullptr;           // stride-2 forward: B origin of the current group of 32 channels
    int fkt = 0, f_left = 0, f_kx = 0, f_ky = 0;
    const int conv_first_shift =
        shifts ? ((p.kbatch / p.conv_kw - 1) * p.conv_wp + (p.conv_kw - 1)) * conv_dil : 0;
    Cursor fcur = first;
    auto f_begin = [&]() {
        const Item it = item_of(fcur);
        ldr_a.init(lda, it.m0, p.M, wave, lane);
        if (!KB && p.n_img != 0) {
            if (shifts && p.n_img < BN) {
                // (implicit convolution over small planes)
                ldr_b.init_folded_many(ldb, it.r0, p.n_img, (p.N - (it.n0 - it.r0)) / p.n_img, (unsigned)p.sB, wave, lane);
            } else {
                const bool has_next = it.n0 - it.r0 + p.n_img < p.N;  // p.N = batches * n_img here
                ldr_b.init_folded(ldb, it.r0, p.n_img, has_next ? (unsigned)p.sB : 0u, wave, lane);
            }
        } else if (KB && p.rows_taps != 0) {
            ldr_b.init_conv_rows(it.n0, p.N, p.rows_taps, p.rows_kw, p.rows_wp, p.rows_plane, p.rows_phase, p.conv_dil, wave, lane);
        } else {
            ldr_b.init(ldb, it.n0, p.N, wave, lane);
        }
        if (taps) {
            // (first channel group of this split: 32 elements along A's rows, 32 planes of B)
            pa = p.A + (long long)it.bz * p.sA + (long long)it.kb0 * BK;
            pb = p.B + (long long)it.bz * p.sB + (long long)it.kb0 * step_b;
        } else {
            pa = p.A + (long long)it.bz * p.sA + (long long)it.kb0 * p.sAk;
            pb = p.B + (long long)it.bz * p.sB + (long long)it.kb0 * p.sBk;
        }
        if (taps) {  // first tap (0, 0): the largest shift (input gradient), or phase (0, 0) unshifted
            pb_group = pb;
            pb += conv_first_shift;
            f_kx = f_ky = 0;
        }
        fkt = 0;
        f_left = it.nt;
    };
    // Past the end of the block's stream the origins stay where they are: the loads that the k loop keeps issuing
    // read the last tile again (into ring slots that nothing reads any more), so that the loop has no "is there a
    // tile left" test in front of every load and one steady wait count.
    auto fetch_advance = [&]() {
        if (!f_valid) return;
        if (--f_left == 0) {
            fw += gdim;
            f_valid = fw < total;
            if (f_valid) {
                cursor_next(fcur);
                f_begin();
            }
        } else if (phases) {
            // Stride-2 forward: all taps of one group of 32 channels in natural order, then the next group.
            if (++fkt == p.kbatch) {
                fkt = 0;
                f_kx = f_ky = 0;
                pa += BK - (long long)(p.kbatch - 1) * p.sAk;
                pb_group += step_b;
                pb = pb_group;
            } else {
                pa += p.sAk;
                if (++f_kx == p.conv_kw) {
                    f_kx = 0;
                    ++f_ky;
                }
                pb = pb_group + (long long)((f_ky & 1) * 2 + (f_kx & 1)) * p.conv_phase + (f_ky >> 1) * p.conv_wp + (f_kx >> 1);
            }
        } else if (taps) {
            // Implicit input gradient: for one group of 32 filters all taps are visited in turn
            // (they read nearly the same rows of B, which stay in the cache), then the next group.
            if (++fkt == p.kbatch) {  // fkt counts taps here
                fkt = 0;
                f_kx = 0;
                pa += BK - (long long)(p.kbatch - 1) * p.sAk;
                pb += step_b + conv_first_shift;  // the last tap has shift 0
            } else {
                pa += p.sAk;
                if (++f_kx == p.conv_kw) {  // next tap: one column to the left, or up a row
                    f_kx = 0;
                    pb += (p.conv_kw - 1 - p.conv_wp) * conv_dil;
                } else {
                    pb -= conv_dil;
                }
            }
        } else if (++fkt == kt_per) {
            fkt = 0;
            pa += wrap_a;
            pb += wrap_b;
        } else {
            pa += step_a;
            pb += step_b;
        }
    };
    // ---- compute stream ----
    // `acc` is the chain the MFMAs add to.  A chain that ran over the whole contraction would grow a
    // rounding error like that of any sequential f32 sum; after every kChainK elements of k it is
    // therefore set aside into `tot` and restarted from zero, which is how a blocked CPU SGEMM
    // (the reference's OpenBLAS) sums as well.
    f32x16 acc[MI][NI], tot[MI][NI];
    constexpr int CHAIN = kChainK / BK;  // k tiles per chain
    auto zero_acc = [&]() {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    };
    auto zero_tot = [&]() {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) tot[i][j][v] = 0.f;
    };
    auto set_aside = [&]() {  // tot += acc, acc = 0
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    tot[i][j][v] += acc[i][j][v];
                    acc[i][j][v] = 0.f;
                }
    };
    auto take_back = [&]() {  // acc += tot
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] += tot[i][j][v];
    };
    // Per-lane float indices of the fragments inside a ring slot.
    int a_idx[KA ? KK : MI], b_idx[KB ? KK : NI];
    {
        const int x = half ^ kc_swizzle<BK>(l31);
        if (KA) {
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) a_idx[kk] = (wm * WM + l31) * BK + (((kk << 1) ^ x) << 2);
        } else {
#pragma unroll
            for (int i = 0; i < MI; ++i) a_idx[i] = half * 4 * BM + ((wm * WM + i * 32 + l31) ^ (half << 5));
        }
        if (KB) {
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) b_idx[kk] = BM * BK + (wn * WN + l31) * BK + (((kk << 1) ^ x) << 2);
        } else {
#pragma unroll
            for (int j = 0; j < NI; ++j) b_idx[j] = BM * BK + half * 4 * BN + ((wn * WN + j * 32 + l31) ^ (half << 5));
        }
    }
    struct Frag {
        float v[4];
    };
    auto read_frags = [&](const float *S, int kk, Frag (&af)[MI], Frag (&bf)[NI]) {
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            if (KA) {
                const float4 t = *reinterpret_cast<const float4 *>(S + a_idx[kk] + i * 32 * BK);
                af[i].v[0] = t.x; af[i].v[1] = t.y; af[i].v[2] = t.z; af[i].v[3] = t.w;
            } else {
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4) af[i].v[s4] = S[a_idx[i] + (kk * 8 + s4) * BM];
            }
        }
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            if (KB) {
                const float4 t = *reinterpret_cast<const float4 *>(S + b_idx[kk] + j * 32 * BK);
                bf[j].v[0] = t.x; bf[j].v[1] = t.y; bf[j].v[2] = t.z; bf[j].v[3] = t.w;
            } else {
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4) bf[j].v[s4] = S[b_idx[j] + (kk * 8 + s4) * BN];
            }
        }
    };
    // SKIP (grouped pair form only): 1 leaves out the 32-row block of parity 0, 2 that of parity 1
    auto mfma_frags = [&](auto skip_c, const Frag (&af)[MI], const Frag (&bf)[NI]) {
        constexpr int SKIP = decltype(skip_c)::value;
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                if (SKIP != 0 && i == SKIP - 1) continue;
#pragma unroll
                for (int j = 0; j < NI; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i].v[s4], bf[j].v[s4], acc[i][j], 0, 0, 0);
            }
    };
    // Returns true when exactly STORES store instructions were issued (interior tile, overwrite).
    auto write_out = [&](const Item &it) -> bool {
        float *Cb;
        long long ldc;
        float alpha, beta;
        if (p.splits > 1) {
            // partial sums: slot it.sp of the workspace, laid out like the output itself for the tap walks
            Cb = p.C + (long long)it.bz * p.sC + (long long)it.sp * p.sCsplit;
            ldc = taps ? p.ldc : p.N;
            alpha = 1.f;
            beta = 0.f;
        } else {
            Cb = p.C + (long long)it.bz * p.sC;
            ldc = p.ldc;
            alpha = p.alpha;
            beta = p.beta;
        }
        if (taps) {
            // implicit input gradient: column -> pixel of the (possibly next) image; the columns
            // of the zero border are dropped
            const int row_base = it.m0 + wm * WM + 4 * half;
            float *dst0[NI];
            bool ok[NI];
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                int col = it.r0 + wn * WN + l31 + j * 32;
                const bool in_range = it.n0 + wn * WN + l31 + j * 32 < p.N;
                long long img = 0;
                if (shifts && p.n_img < BN) {  // small planes: the tile covers several images
                    const int q = col / p.n_img;
                    col -= q * p.n_img;
                    img = q * p.sC;
                } else if (col >= p.n_img) {
                    col -= p.n_img;
                    img = p.sC;
                }
                const int iy = col / p.conv_wp, ix = col - iy * p.conv_wp;
                ok[j] = in_range && ix < p.conv_w;
                dst0[j] = p.conv_pair_w != 0 ? Cb + img + (long long)(2 * iy + p.conv_pair_a) * p.conv_pair_w + 2 * ix
                                             : Cb + img + iy * p.conv_w + ix;
            }
            if (grouped) {
                // the wave's first 32-row block is parity 0 of 32 channels, its second block parity 1 of the same
                // channels: value v of the two blocks are neighbours in memory
                if constexpr (MI == 2) {
                    const int ch_base = (it.m0 + wm * WM) / 2 + 4 * half;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int ch = ch_base + 8 * (v / 4) + (v % 4);
#pragma unroll
                        for (int j = 0; j < NI; ++j)
                            if (ok[j] && 2 * ch < p.M) {
                                float2 *dst = reinterpret_cast<float2 *>(dst0[j] + (long long)ch * ldc);
                                *dst = make_float2(alpha * acc[0][j][v], alpha * acc[1][j][v]);
                            }
                    }
                }
                return false;
            }
            if (p.conv_pair_w != 0) {
                // rows come in (channel, parity) pairs: a lane's values v, v + 1 (v even) are the two column
                // parities of one channel at neighbouring addresses
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int v = 0; v < 16; v += 2) {
                        const int row = row_base + i * 32 + 8 * (v / 4) + (v % 4);
#pragma unroll
                        for (int j = 0; j < NI; ++j)
                            if (ok[j] && row < p.M) {
                                float2 *dst = reinterpret_cast<float2 *>(dst0[j] + (long long)(row >> 1) * ldc);
                                *dst = make_float2(alpha * acc[i][j][v], alpha * acc[i][j][v + 1]);
                            }
                    }
                return false;
            }
            // rows outermost: the segments of one output row leave back to back, so the cache lines
            // they share are completed before they can be evicted
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = row_base + i * 32 + 8 * (v / 4) + (v % 4);
#pragma unroll
                    for (int j = 0; j < NI; ++j)
                        if (ok[j] && row < p.M) {
                            float *dst = dst0[j] + (long long)row * ldc;
                            const float r = alpha * acc[i][j][v];
                            *dst = beta == 0.f ? r : r + beta * *dst;
                        }
                }
            return false;
        }
        const bool full = it.m0 + BM <= p.M && it.n0 + BN <= p.N;
        const int row_base = it.m0 + wm * WM + 4 * half;
        // column inside batch it.bz; a folded tile may run on into the next batch, whose columns
        // sit sC - n_img elements further
        const int col_base = (p.n_img != 0 ? it.r0 : it.n0) + wn * WN + l31;
        const int col_end = p.n_img != 0 ? p.n_img : p.N;
        const long long next_img = p.sC - p.n_img;
        if (full && beta == 0.f) {
            // interior tile, overwrite: straight stores
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j) {
                    const int col = col_base + j * 32;
                    float *dst = Cb + (long long)(row_base + i * 32) * ldc + col + (col >= col_end ? next_img : 0);
#pragma unroll
                    for (int v = 0; v < 16; ++v)  // written once, read by a later kernel: streaming stores
                        st_stream(dst + (long long)(8 * (v / 4) + (v % 4)) * ldc, alpha * acc[i][j][v]);
                }
            return true;
        } else {
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j) {
                    const int col = col_base + j * 32;
                    // beyond the operand: past N, or (folded) past the last batch
                    const bool col_ok = p.n_img != 0 ? it.n0 + wn * WN + l31 + j * 32 < p.N : col < p.N;
                    const long long shift = col >= col_end ? next_img : 0;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int row = row_base + i * 32 + 8 * (v / 4) + (v % 4);
                        if (row < p.M && col_ok) {
                            float *dst = Cb + (long long)row * ldc + col + shift;
                            const float r = alpha * acc[i][j][v];
                            *dst = beta == 0.f ? r : r + beta * *dst;
                        }
                    }
                }
        }
        return false;
    };

    Frag af[2][MI], bf[2][NI];
    unsigned fill_addr = lds_wave;  // LDS byte address (this wave's share) of the slot being filled
    auto second_half = [&](auto skip_c, const float *cur, const float *nxt, bool last) {
        constexpr int SKIP = decltype(skip_c)::value;
        constexpr int MIA = SKIP != 0 ? MI - 1 : MI;        // 32-row blocks that multiply
        constexpr int NM = (KK - KK / 2) * 4 * MIA * NI;  // MFMAs in this half
        constexpr int SPACING = NM / L;                   // MFMAs between two loads
        static_assert(SPACING >= 1, "more loads than MFMAs");
#pragma unroll
        for (int kk = KK / 2; kk < KK; ++kk) {
            if (kk + 1 < KK) read_frags(cur, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
            else if (!last) read_frags(nxt, 0, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
                for (int i = 0; i < MI; ++i) {
                    if (SKIP != 0 && i == SKIP - 1) continue;
                    const int ia = SKIP == 1 ? i - 1 : i;  // index among the blocks that multiply
#pragma unroll
                    for (int j = 0; j < NI; ++j) {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[kk & 1][i].v[s4], bf[kk & 1][j].v[s4],
                                                                         acc[i][j], 0, 0, 0);
                        const int m = (((kk - KK / 2) * 4 + s4) * MIA + ia) * NI + j;
                        const int load = m / SPACING;
                        if (m % SPACING == SPACING - 1 && load < L) {
                            __builtin_amdgcn_sched_barrier(0);
                            if (load < LoadA::PER_WAVE) ldr_a.issue_one(load, pa, fill_addr);
                            else ldr_b.issue_one(load - LoadA::PER_WAVE, pb, fill_addr + BM * BK * 4u);
                            if (load == L - 1) fetch_advance();
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // Prologue: tiles 0 .. STAGES-2 of the stream.
    f_begin();
#pragma unroll
    for (int st = 0; st < STAGES - 1; ++st) {
        ldr_a.template issue<0, 8>(pa, fill_addr);
        ldr_b.template issue<0, 8>(pb, fill_addr + BM * BK * 4u);
        fetch_advance();
        fill_addr += TILE * 4u;
    }
    wait_loads_then_barrier<(STAGES - 2) * L>();

    unsigned cw = bid;
    Cursor ccur = first;
    Item ci = item_of(ccur);
    const float *cur = lds;  // ring slot being multiplied
    const float *const ring_end = lds + STAGES * TILE;
    read_frags(cur, 0, af[0], bf[0]);

    bool after_epilogue = false;
    while (true) {  // work items of this block
        zero_acc();
        int c_left = ci.nt;
        const bool chained = ci.nt > CHAIN + CHAIN / 4;  // more than one chain: their sums meet in `tot`
        if (chained) zero_tot();
        int chain_left = CHAIN;
        const bool last_item = cw + gdim >= total;
        int c_tap = 0;  // (grouped pair form) tap slot of the k tile being multiplied; an item starts at slot 0
        do {  // k tiles of the item: within a chain the accumulators are touched by MFMAs only
            const bool last = c_left == 1 && last_item;  // nothing follows in the stream
            const float *nxt = cur + TILE == ring_end ? lds : cur + TILE;
            // which parity, if any, has no filter tap at this slot (wave-uniform)
            int skip = 0;
            if (grouped) {
                skip = (p.conv_pair_skip[0] >> c_tap) & 1u ? 1 : ((p.conv_pair_skip[1] >> c_tap) & 1u ? 2 : 0);
                if (++c_tap == p.kbatch) c_tap = 0;
            }
            auto first_half = [&](auto skip_c) {
#pragma unroll
                for (int kk = 0; kk < KK / 2; ++kk) {
                    read_frags(cur, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
                    __builtin_amdgcn_sched_barrier(0);  // all fragment reads of the next group go out first
                    mfma_frags(skip_c, af[kk & 1], bf[kk & 1]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            // first half of the tile's k range
            if (grouped && skip == 1) first_half(std::integral_constant<int, grouped ? 1 : 0>{});
            else if (grouped && skip == 2) first_half(std::integral_constant<int, grouped ? 2 : 0>{});
            else first_half(std::integral_constant<int, 0>{});
            // The next tile must have landed; tiles further ahead may still be in flight.
            if (after_epilogue) wait_loads_then_barrier<AFTER_EPILOGUE>();
            else wait_loads_then_barrier<STEADY>();
            after_epilogue = false;
            // Every wave has left the previous tile's slot.  Its loads are issued one at a time
            // between the MFMAs of the rest of this tile: a clump of loads would leave the matrix
            // pipe idle while the wave issues them, and all waves of the block would queue at the
            // address unit right after the barrier.
            if (grouped && skip == 1) second_half(std::integral_constant<int, grouped ? 1 : 0>{}, cur, nxt, last);
            else if (grouped && skip == 2) second_half(std::integral_constant<int, grouped ? 2 : 0>{}, cur, nxt, last);
            else second_half(std::integral_constant<int, 0>{}, cur, nxt, last);
            fill_addr = fill_addr + TILE * 4u == lds_wave + STAGES * TILE * 4u ? lds_wave : fill_addr + TILE * 4u;
            cur = nxt;
            if (--chain_left == 0 && c_left - 1 > CHAIN / 4) {
                // (a remainder of up to a quarter chain joins the chain before it: the 576-element
                // contractions of a 3x3 convolution over 64 channels stay one chain)
                set_aside();
                chain_left = CHAIN;
            }
        } while (--c_left != 0);
        if (chained) take_back();
        const bool counted = write_out(ci);
        if (last_item) {
            // the loads issued past the end of the stream must land before the block gives up its LDS
            asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
            break;
        }
        after_epilogue = counted;
        cw += gdim;
        cursor_next(ccur);
        ci = item_of(ccur);
    }
}

template <int BM, int BN, int BK, int WM, int WN, int STAGES, bool KA, bool KB, int CONV>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64, 1) void gemm_dl_kernel(GemmParams p)
{
    gemm_dl_body<BM, BN, BK, WM, WN, STAGES, KA, KB, CONV>(p, blockIdx.x, gridDim.x);
}

// Two products of one tile shape in one launch: blocks [0, grid0) work through the items of the first, the others
// through those of the second.  A CU whose block of the first product has run out of items takes a block of the second
// at once, where two launches leave it idle until the first has drained everywhere (the two row parities of the
// stride-2 input gradient: two or three rounds of tiles each).
struct DualParams {
    GemmParams q[2];
    unsigned grid0;
};
template <int BM, int BN, int BK, int WM, int WN, int STAGES, bool KA, bool KB, int CONV>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64, 1) void gemm_dl_dual_kernel(DualParams d)
{
    const bool second = blockIdx.x >= d.grid0;
    gemm_dl_body<BM, BN, BK, WM, WN, STAGES, KA, KB, CONV>(d.q[second ? 1 : 0], blockIdx.x - (second ? d.grid0 : 0u),
                                                           second ? gridDim.x - d.grid0 : d.grid0);
}

static long long dl_grid(const GemmParams &p, int cus, int blocks_per_cu)
{
    long long g = (long long)cus * (blocks_per_cu > 0 ? blocks_per_cu : 1);
    if (g >= p.total_blocks) g = p.total_blocks;        // one item per block
    else g = g >= kXcds ? g - g % kXcds : kXcds;         // the kernel steps items by grid / 8
    return g;
}

template <int BM, int BN, int BK, int WM, int WN, int STAGES>
static void launch_dl(hipStream_t st, bool ka, bool kb, const GemmParams &p, int cus, int blocks_per_cu, const GemmParams *second)
{
    constexpr int NT = (BM / WM) * (BN / WN) * 64;
    if (second != nullptr) {
        // two grouped pair-form products in one launch (the caller has checked that the tile is one of those)
        if constexpr (WM == 64 && BM % 64 == 0) {
            DualParams d;
            d.q[0] = p;
            d.q[1] = *second;
            const long long g0 = dl_grid(p, cus, blocks_per_cu), g1 = dl_grid(*second, cus, blocks_per_cu);
            d.grid0 = (unsigned)g0;
            hipLaunchKernelGGL((gemm_dl_dual_kernel<BM, BN, BK, WM, WN, STAGES, true, false, 5>), dim3((unsigned)(g0 + g1)), dim3(NT), 0,
                               st, d);
        }
        return;
    }
#define AG_GEMM_DL_CASE(KA_, KB_)                                                                     \
    if constexpr ((KA_ || BM % 64 == 0) && (KB_ || BN % 64 == 0)) if (ka == KA_ && kb == KB_) {      \
        auto kern = gemm_dl_kernel<BM, BN, BK, WM, WN, STAGES, KA_, KB_, 3>;                              \
        if constexpr (KA_ && !KB_) /* the implicit convolution over filter taps */                    \
            if (p.conv_phase != 0) kern = gemm_dl_kernel<BM, BN, BK, WM, WN, STAGES, KA_, KB_, 4>;       \
            else if (p.conv_pair_grouped != 0) {                                                      \
                if constexpr (WM == 64) kern = gemm_dl_kernel<BM, BN, BK, WM, WN, STAGES, KA_, KB_, 5>;  \
            } else if (p.conv_wp != 0)                                                                \
                kern = p.conv_dil != 1 ? gemm_dl_kernel<BM, BN, BK, WM, WN, STAGES, KA_, KB_, 2>         \
                                       : gemm_dl_kernel<BM, BN, BK, WM, WN, STAGES, KA_, KB_, 1>;        \
        hipLaunchKernelGGL(kern, dim3((unsigned)dl_grid(p, cus, blocks_per_cu)), dim3(NT), 0, st, p);  \
        return;                                                                                       \
    }
    AG_GEMM_DL_CASE(true, true)
    AG_GEMM_DL_CASE(true, false)
    AG_GEMM_DL_CASE(false, true)
    AG_GEMM_DL_CASE(false, false)
#undef AG_GEMM_DL_CASE
}

// `second` != null: a second grouped pair-form product (GemmParams::conv_pair_grouped) of the same tile, carried by the
// same launch; only for the tiles whose waves hold 64 rows (configurations 13, 14, 15 and 18).
void launch_direct(hipStream_t st, int cfg, bool ka, bool kb, const GemmParams &p, int cus, int blocks_per_cu,
                   const GemmParams *second)
{
    if (second != nullptr && !(ka && !kb && p.conv_pair_grouped != 0 && second->conv_pair_grouped != 0 &&
                               ((cfg >= 13 && cfg <= 15) || cfg == 18))) {
        // not a pair of products that one launch can carry: one after the other
        launch_direct(st, cfg, ka, kb, p, cus, blocks_per_cu, nullptr);
        launch_direct(st, cfg, ka, kb, *second, cus, blocks_per_cu, nullptr);
        return;
    }
    switch (cfg) {
        //                BM   BN  BK   WM  WN STAGES
        case 13: launch_dl<128, 128, 32, 64, 64, 3>(st, ka, kb, p, cus, blocks_per_cu, second); break;
        case 14: launch_dl<128, 256, 32, 64, 64, 3>(st, ka, kb, p, cus, blocks_per_cu, second); break;
        case 15: launch_dl<256, 128, 32, 64, 64, 3>(st, ka, kb, p, cus, blocks_per_cu, second); break;
        case 16: launch_dl<192, 128, 32, 96, 32, 3>(st, ka, kb, p, cus, blocks_per_cu, nullptr); break;
        case 17: launch_dl<128, 192, 32, 32, 96, 3>(st, ka, kb, p, cus, blocks_per_cu, nullptr); break;
        case 18: launch_dl<128, 64, 32, 64, 32, 3>(st, ka, kb, p, cus, blocks_per_cu, second); break;
        // small problems: tiles that still give every CU a block or two
        // (32 rows only with a k-contiguous A: an m-contiguous tile is swizzled in groups of 64 rows)
        case 20: launch_dl<32, 128, 32, 32, 32, 3>(st, ka, kb, p, cus, blocks_per_cu > 0 ? blocks_per_cu : 2, nullptr); break;
        case 21: launch_dl<64, 64, 32, 32, 32, 3>(st, ka, kb, p, cus, blocks_per_cu > 0 ? blocks_per_cu : 2, nullptr); break;
        default: launch_dl<64, 128, 32, 32, 64, 3>(st, ka, kb, p, cus, blocks_per_cu > 0 ? blocks_per_cu : 2, nullptr); break;
    }
}

}  // namespace ag
