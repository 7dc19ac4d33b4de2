// Several W8A8 contractions in ONE launch: a workgroup per compute unit walks a list of output tiles, and the K
// stages of all its tiles form one uninterrupted stream.
//   acc[m,n] = sum_k qx[m,k] * qw[n,k],   y = ((float)acc * sx[m]) * sw[n]      (per problem of the batch)
//
// Why.  A prefill GEMM launched on its own spends a third of its time outside the stage loop: the gap to the
// previous kernel, the first memory round trip of 256 workgroups asking at once, and an epilogue in which the matrix
// pipe idles while 196 KB per compute unit are converted and stored.  Its tile shape is also dictated by how the
// tile count divides by the number of compute units.  Here
//   - the tiles of all problems form one work list of 256 x 256 tiles, balanced as a whole on the host;
//   - the direct-to-LDS loads run two stages ahead of the matrix instructions ACROSS tile boundaries (the stage
//     buffers rotate for the whole life of the workgroup and never drain between tiles);
//   - a wave owns 64 x 128 outputs over the WHOLE of K (128 accumulation registers), so no partial sums are
//     exchanged between waves: when a tile's last stage has been issued the wave converts, scales, stores and clears
//     its 32 accumulators in one straight run of vector instructions, while the loads of the next tile (requested
//     two stages ago) are already landing.
//     (The tile is as large as the unit's LDS allows: two activation and three weight stage buffers of 32 KB fill its
//     160 KB.  Against 256 x 192 tiles it moves a tenth fewer bytes from LDS and a seventh fewer from L2 per matrix
//     instruction, and the matrix pipe of this part runs against a power limit that every byte moved lowers:
//     measured 3 to 4 % faster on the four prefill projections, although the coarser tiles balance a little worse.)
//     (Measured and not kept: a second accumulator set, drained one accumulator per stage under the next tile's
//     matrix instructions.  Both waves of a SIMD reach the drain at the same point of a stage, so the matrix pipe
//     idles all the same, and the store queues behind the stage's direct-to-LDS loads on the unit's one memory path:
//     it cost 1,000 ticks per stage, more than the straight run at the end of the tile.)
// A tile that would cross the edge of its matrix is moved inwards until it fits: the overlap with its neighbour
// is computed twice, both times to the same values (exact integers, the same fp32 operations), so every problem
// needs only M >= 256, N >= 256; no ragged code path exists.
//
// Waves: 8 = 4 (rows) x 2 (columns), two per SIMD; wave tile 4 x 8 matrix-instruction tiles.  A 128-byte K stage
// is two halves of 64 bytes; a half is eight groups (one weight fragment against the four activation fragments).
// LDS layout, swizzle and load shapes are those of gemm_pair.hip.  Per wave and half: 8 weight and 4 activation
// fragment reads, all of them requested half a stage before they are used (see the stage below), and ONE barrier
// a stage.
//
// Registers: v[128..255] are the accumulators and v[104..127] hold the scales of the wave's rows and columns for
// the tile in work (LDS has no room for them), all named by hand; the kernel is limited to v0..v103 for everything
// the compiler places (see gemm_pair_ops.h): fragments for two K halves and the addresses.
//
// Memory operations complete in issue order (one counter for loads and stores), and every wait below is written
// against that order.  Every wave issues an eighth of the loads and stores its own results.
//
// The list itself is made on the host when the batch is created (rounds of compact patches of the tile grid, one
// patch per XCD and round, longest K first: see build_lists) and lives in device memory.
//
// Bound: int8 MFMA (2*M*N*K ops per problem).  Exact integer arithmetic.
#include <string.h>

#include <algorithm>
#include <atomic>
#include <new>
#include <vector>

#include "common.h"
#include "gemm_pair_ops.h"

#ifndef MI_STORE_MOD
#define MI_STORE_MOD " nt"   // the results are not read again by this kernel: stores that do not displace the operands in L2 (measured: 385 -> 363 us for the four prefill projections as one batch)
#endif

namespace mi {
namespace list {

using namespace pair;

constexpr int MAX_PROBLEMS = 8;
constexpr int MAX_TILES = 1 << 20;

struct Problem {
    const int8_t *qx, *qw;
    const float *sx, *sw;
    void *out;   // fp32 [M,N] (dequantized) or int32 [M,N]
    int M, N, K, pad;
};
struct Batch {
    Problem p[MAX_PROBLEMS];
};

struct Cfg {
    static constexpr int TM = 4, TN = 8;                // matrix-instruction tiles of a wave
    static constexpr int BM = 256, BN = 256;            // 4 x 2 waves
    static constexpr int NBX = BM / 8, NBW = BN / 8;    // 1 KB blocks (8 rows x 128 B) per stage
    static constexpr int XSTAGE = NBX * 1024, WSTAGE = NBW * 1024, XAREA = 2 * XSTAGE;
    static constexpr int LDS = XAREA + 3 * WSTAGE;      // two activation buffers, three weight buffers
    static constexpr int LX = NBX / 8, LW = NBW / 8;    // loads of a wave per stage
    static constexpr int NACC = TM * TN;                // accumulators of a set
    // a lane's scales for its wave's tile: of rows r % 8 and 8 + r % 8 of each of the TM row tiles (v[SCL0 + 2i],
    // v[SCL0 + 2i + 1]), and four column scales for each pair of column tiles (v[SCL0 + 2 TM + 4 jp ..])
    static constexpr int NSCL = 2 * TM + 4 * (TN / 2), SCL0 = vacc::ACC0 - NSCL;
    static constexpr int LSCL = 2 * TM + TN / 2;        // loads that bring them, per wave and tile
    static constexpr int MIN_STAGES = 3;                // the loads run up to three stages ahead, into the next tile at most
    static_assert(LX <= TM && LW <= TN && TN >= TM + 2, "where the stage issues its loads and what its waits count");
    static_assert(vacc::ACC0 + 4 * NACC <= 256, "the accumulators lie above the compiler's registers");
    static_assert(LDS <= 160 * 1024, "LDS of a compute unit");
};

#ifdef MI_GEMM_TIMELINE
// The measurement build keeps a few more scalars alive and may spill some: a base the compiler brings back with a
// vector instruction needs five wait states before a memory instruction reads it (see the build check of the
// product library, which allows no such spill); here every load pays them.
__device__ __forceinline__ void dma16(const int8_t *sbase, unsigned voff, unsigned ldsaddr)
{
    asm volatile("s_nop 4" ::: "memory");
    pair::dma16(sbase, voff, ldsaddr);
}
#endif
#ifdef MI_GEMM_TIMELINE
// Built only into libmi355_int8_timeline.so (bench.py --gemm-timeline): wave 0 of every workgroup leaves, per tile,
// the clock ticks (s_memtime) and the 100 MHz real time at which the tile's first and last stage began and ended.
#ifndef MI_TL_WAVE
#define MI_TL_WAVE 0
#endif
constexpr int TL_WGS = 512, TL_TILES = 16;
__device__ unsigned long long g_list_timeline[TL_WGS * TL_TILES * 8];
#endif

__device__ __forceinline__ v4i sload4(const v4i *p)
{
    v4i v;
    asm volatile("s_load_dwordx4 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(p) : "memory");
    return v;
}
// lane-derived values are recomputed where they are needed from a copy of the lane number that the compiler
// cannot see through: otherwise it computes all of them once, before the tile loop, and 64 registers cannot hold
// them beside the fragments
__device__ __forceinline__ int opaque(int v)
{
    asm volatile("" : "+v"(v));
    return v;
}
// a + s in place, where the compiler would otherwise keep one register per value that s takes
__device__ __forceinline__ unsigned add_vs(unsigned a, unsigned s)
{
    unsigned r;
    asm volatile("v_add_u32 %0, %1, %2" : "=v"(r) : "s"(s), "v"(a));
    return r;
}
// the scales of rows (r % 8) and (8 + r % 8) of a 16-row tile into v[R], v[R + 1]; four column scales into v[R .. R + 3]
template <int R, int OFF>
__device__ __forceinline__ void scale_load_pair(unsigned voff, const float *sbase)
{
#ifdef MI_GEMM_TIMELINE
    asm volatile("s_nop 4" ::: "memory");   // (a scalar base brought back from a spill: see dma16 above)
#endif
    asm volatile("global_load_dword v%c2, %0, %1 offset:%c4\n\tglobal_load_dword v%c3, %0, %1 offset:%c5"
                 :
                 : "v"(voff), "s"(sbase), "n"(R), "n"(R + 1), "n"(OFF), "n"(OFF + 32)
                 : "memory");
}
template <int R, int OFF>
__device__ __forceinline__ void scale_load4(unsigned voff, const float *sbase)
{
#ifdef MI_GEMM_TIMELINE
    asm volatile("s_nop 4" ::: "memory");
#endif
    asm volatile("global_load_dwordx4 v[%c2:%c3], %0, %1 offset:%c4" : : "v"(voff), "s"(sbase), "n"(R), "n"(R + 3), "n"(OFF) : "memory");
}
template <int R>
__device__ __forceinline__ float scale_reg()
{
    float v;
    asm volatile("v_mov_b32 %0, v%c1" : "=v"(v) : "n"(R));
    return v;
}

template <bool DEQ>
__global__ __launch_bounds__(512) __attribute__((amdgpu_num_vgpr(Cfg::SCL0 / 2))) void k_w8a8_list(
    const Batch bt, const v4i *__restrict__ lists, int per_wg)
{
    using C = Cfg;
    constexpr int TM = C::TM, TN = C::TN;
    constexpr int XSTAGE = C::XSTAGE, WSTAGE = C::WSTAGE, XAREA = C::XAREA;
    constexpr int NACC = C::NACC;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    // v[128 .. 255] are this kernel's accumulators and v[104 .. 127] its scales, named by hand: the attribute above
    // keeps everything the compiler places below v104, and this clobber makes the wave's register count cover them
    asm volatile("" ::: "v104", "v255");
    static_assert(C::SCL0 == 104 && vacc::ACC0 == 128, "the clobber above names the first register by hand");

    const int tid = threadIdx.x, lane0 = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;   // wave tile: rows wm*64.., columns wn*128..
    const unsigned lds_base = (unsigned)(uintptr_t)(lptr_t)smem;
    const unsigned lds_x = lds_base + wave * 1024, lds_w = lds_base + XAREA + wave * 1024;

    const v4i *const my = lists + (int64_t)blockIdx.x * per_wg;
    // {problem or -1, first row, first column, -}: the tile the matrix pipe works on (three scalars, not the entry's four)
    int e_p, e_m0, e_n0;
    {
        const v4i e = sload4(my);
        e_p = e[0];
        e_m0 = e[1];
        e_n0 = e[2];
    }
    if (e_p < 0) return;
    // the scales of the tile's rows and columns (fetched where the tile is entered: a scalar load inside the stage
    // would have to wait for every LDS read in flight with it)
    const float *e_sx = bt.p[e_p].sx + e_m0, *e_sw = bt.p[e_p].sw + e_n0;

    // ---- load side.  The load cursor (a tile and a stage of it) runs two stages ahead of the matrix instructions.
    // lane l = 8*rho + c fetches the 16-byte chunk c ^ sigma of row rho of a block; wave w fills blocks w + 8q of
    // a stage (four of the activations, four of the weights): every wave issues the same share of the loads, and
    // one lane offset serves every block of a tile: base of the tile (two scalars) + this lane's offset + a scalar
    // that moves with q and with the stage (one scalar and one vector addition a load; 64-bit scalar address
    // arithmetic for every load, on four waves only, made those four waves the last at every barrier by 500 ticks)
    const int8_t *lx = nullptr, *lw = nullptr;
    unsigned lbstep = 0;
    unsigned lvoff = 0;
    int lkt = 0, lnk = 0;
    bool ldv = false;   // the cursor stands on a stage that exists
    auto cursor_to = [&](const v4i &e) {
        const Problem &P = bt.p[e[0]];
        const int K = P.K;
        lnk = K >> 7;
        lkt = 0;
        lx = P.qx + (int64_t)e[1] * K;
        lw = P.qw + (int64_t)e[2] * K;
        lbstep = 64u * (unsigned)K;   // eight blocks of eight rows
        const int l = opaque(lane0);
        const int lrow = wave * 8 + (l >> 3);
        const unsigned lchunk = (unsigned)(((l & 7) ^ (((wave & 1) << 2) | (l >> 4))) << 4);
        lvoff = (unsigned)lrow * (unsigned)K + lchunk;
        ldv = true;
    };
    auto issue_x = [&](auto I, unsigned buf) {   // part p of the cursor's stage
        constexpr int p_ = decltype(I)::value;
        dma16(lx, add_vs(lvoff, (unsigned)lkt * 128u + p_ * lbstep), lds_x + buf + p_ * 8192);
    };
    auto issue_w = [&](auto I, unsigned buf) {
        constexpr int p_ = decltype(I)::value;
        dma16(lw, add_vs(lvoff, (unsigned)lkt * 128u + p_ * lbstep), lds_w + buf + p_ * 8192);
    };

    // ---- read side: fragment (16 rows, 64 K bytes): lane (r = l%16, g = l/16) reads row r, chunk 4*half + g
    v4i xa[TM], xc[TM], w[TN];   // activation fragments of a first / second K half, weight fragments
    unsigned xo0 = 0, xo1 = 0, wo0 = 0, wo1 = 0;   // this lane's fragment addresses in buffer 0, K half 0 / 1
    {
        const int l = opaque(lane0);
        const int r = l & 15, g_ = l >> 4;
        const int rho = r & 7, bpar = r >> 3;
        const int sigma = (bpar << 2) | (rho >> 1);
        const unsigned roff0 = bpar * 1024 + ((8 * rho + ((0 + g_) ^ sigma)) << 4);
        const unsigned roff1 = bpar * 1024 + ((8 * rho + ((4 + g_) ^ sigma)) << 4);
        xo0 = lds_base + wm * TM * 2048 + roff0;
        xo1 = lds_base + wm * TM * 2048 + roff1;
        wo0 = lds_base + XAREA + wn * TN * 2048 + roff0;
        wo1 = lds_base + XAREA + wn * TN * 2048 + roff1;
    }
    // stage s of the stream lives in activation buffer s % 2 and weight buffer s % 3, for the whole life of the workgroup
    unsigned xcur = 0, xnxt = XSTAGE, wcur = 0, wnxt = WSTAGE, wnn = 2 * WSTAGE;

    // ---- the tile being computed
    int kt = 0, nk = 0;
    bool first_tile = true;   // no stores of a tile before this one are in flight

    // one stage.  There is ONE copy of this code in the source and one loop around it: a fragment register is written
    // by an LDS read the compiler cannot follow (its data arrives later), so no value of xa / xc / w may ever have to
    // be moved where two paths of the control flow meet.  The last stage of a workgroup therefore also requests "next"
    // fragments (from a buffer that holds nothing new; they are never used).  (The compiler may still duplicate the
    // body, and does: it peels a tile's first stage off the loop.  That is harmless as long as every fragment keeps
    // its registers from one copy to the next; the build reads the assembly and stops if a fragment register is ever
    // the source of a move or if the LDS reads write more register ranges than there are fragments.)
    //
    // Fragments are requested half a stage ahead: while the eight groups of a K half run, the four activation
    // fragments of the next half arrive in the other activation set (xa: first halves, xc: second halves) and weight
    // fragment k of the next half is requested into w[k] right behind group k, the last reader of the old w[k].
    // One barrier a stage, behind the first group of the second half: by then every read of this stage's buffers has
    // been issued (the second half's fragments during the first half) and, at the barrier, has landed; behind it the
    // next stage's buffers are read, the activation buffer takes the loads of stage + 2, and the weight buffer is
    // free for the stage after that (its loads are issued during the next stage's first half).
#ifdef MI_GEMM_TIMELINE
    unsigned tl_wait = 0, tl_bar = 0;   // ticks of a tile spent in the wait in front of the barrier / in the barrier
    unsigned tl_wait1 = 0;              // ... of which in the tile's second stage
#endif
    // The scales of the tile in work, requested in its first stage: 2 TM single row scales and TN / 2 groups of four
    // column scales per lane, into v[SCL0 ..].  They are read when the tile's last stage has been issued: a tile has
    // at least three stages, and the wait in front of the second stage's barrier already covers these loads.
    auto load_scales = [&]() {
        const float *bx = e_sx, *bw = e_sw;
        const int l = opaque(lane0);
        const int r = l & 15, g_ = l >> 4;
        const unsigned vx = (unsigned)((wm * 64 + (r & 7)) * 4);
        const unsigned vw = (unsigned)((wn * (16 * TN) + (r < 8 ? 0 : 16) + 4 * g_) * 4);
        static_for<TM>([&](auto I) {
            constexpr int i = decltype(I)::value;
            scale_load_pair<C::SCL0 + 2 * i, 64 * i>(vx, bx);
        });
        static_for<TN / 2>([&](auto JP) {
            constexpr int jp = decltype(JP)::value;
            scale_load4<C::SCL0 + 2 * TM + 4 * jp, 128 * jp>(vw, bw);
        });
    };
    auto stage = [&]() {
        const bool ld = ldv;
        using I0 = std::integral_constant<int, 0>;
        using I1 = std::integral_constant<int, 1>;
        using I2 = std::integral_constant<int, 2>;
        using I3 = std::integral_constant<int, 3>;
        // ---- K half 0 (fragments xa, w).  In flight, oldest first, from the stage before:
        //      W0 | x0 W1 | x1 W2 | x2 W3 | x3 W4 | W5 | W6 | W7
        {
            const unsigned ax1 = add_vs(xo1, xcur), aw1 = add_vs(wo1, wcur);
            static_for<TN>([&](auto J) {
                constexpr int j = decltype(J)::value;
                if constexpr (j < TM) ds_read128<j * 2048>(xc[j], ax1);
                if constexpr (j < C::LW) {
                    if (ld) issue_w(J, wnn);
                }
                // x0..x3 and W0..W3 are in; W4..W7 and the read above may not be
                if constexpr (j == 0) wait_lgkm<TN - TM + 1>();
                // Wj is in: the 2 TM reads of this half's first TM groups and the TN - TM - 1 weight fragments
                // requested last (of this half behind it, of the next half before it) are younger
                if constexpr (j >= TM) wait_lgkm<TN + TM - 1>();
                if constexpr (j == C::LW) {
                    if (kt == 0) {   // this tile's scales, for the end of the tile, into their registers
                        if constexpr (DEQ) load_scales();
                    }
                }
                if (kt == 0) {   // a tile's first instruction on an accumulator sets it: nothing is cleared between tiles
                    static_for<TM>([&](auto I) {
                        vacc::mfma_set<4 * (j * TM + decltype(I)::value)>(w[j], xa[decltype(I)::value]);
                    });
                } else {
                    static_for<TM>([&](auto I) {
                        vacc::mfma_acc<4 * (j * TM + decltype(I)::value)>(w[j], xa[decltype(I)::value]);
                    });
                }
                ds_read128<j * 2048>(w[j], aw1);   // w[j] has been read for the last time
            });
        }
        // ---- K half 1 (fragments xc, w).  In flight: x0 W0 | x1 W1 | x2 W2 | x3 W3 | W4 | W5 | W6 | W7
        {
            wait_lgkm<TN - TM + 1>();   // x0..x3 and W0..W2 are in
            static_for<TM>([&](auto I) { vacc::mfma_acc<4 * decltype(I)::value>(w[0], xc[decltype(I)::value]); });
            // The barrier.  Every read of this stage's buffers has landed in this wave, and a loading wave's share of
            // the next stage as well.  Memory operations complete in order; issued since the last load of the next
            // stage (its fourth activation part, in the stage before): in a tile's first stage the NACC stores of
            // the tile before it; this stage's four weight parts; in a tile's first stage the loads of its scales.
#ifdef MI_GEMM_TIMELINE
            const unsigned tl_s0 = (unsigned)__builtin_amdgcn_s_memtime();
#endif
            {
                constexpr int SC = DEQ ? C::LSCL : 0, LW = C::LW;
                if (!ldv) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                else if (kt == 0 && !first_tile) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(LW + SC + NACC) : "memory");
                else if (kt == 0) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(LW + SC) : "memory");
                else asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(LW) : "memory");
            }
#ifdef MI_GEMM_TIMELINE
            const unsigned tl_s1 = (unsigned)__builtin_amdgcn_s_memtime();
#endif
            __builtin_amdgcn_s_barrier();
#ifdef MI_GEMM_TIMELINE
            tl_wait += tl_s1 - tl_s0;
            if (kt == 1 && !first_tile) tl_wait1 = tl_s1 - tl_s0;   // the first wait that has to see the previous tile's stores acknowledged
            tl_bar += (unsigned)__builtin_amdgcn_s_memtime() - tl_s1;
#endif
            const unsigned nax0 = add_vs(xo0, xnxt), naw0 = add_vs(wo0, wnxt);
            ds_read128<0>(w[0], naw0);
            static_for<TN - 1>([&](auto J1) {
                constexpr int j = decltype(J1)::value + 1;
                if constexpr (j - 1 < TM) {
                    ds_read128<(j - 1) * 2048>(xa[j - 1], nax0);
                    if (ld) issue_x(std::integral_constant<int, j - 1>{}, xcur);
                }
                static_for<TM>([&](auto I) {
                    vacc::mfma_acc<4 * (j * TM + decltype(I)::value)>(w[j], xc[decltype(I)::value]);
                });
                ds_read128<j * 2048>(w[j], naw0);
            });
        }
        {
            const unsigned t = xcur; xcur = xnxt; xnxt = t;
            const unsigned u = wcur; wcur = wnxt; wnxt = wnn; wnn = u;
        }
    };
    static_assert(C::LW + C::LSCL + NACC + C::LX <= 63, "the memory counter has six bits");

    // The tile's accumulators leave: converted, scaled by the row and the column scale, stored and cleared for the
    // next tile; accumulator (j, i) is named at compile time.  Two neighbouring column tiles are paired and swap
    // halves between lanes r and r ^ 8, so that a store instruction writes 8 rows x 128 B: whole cache lines
    // (stores of 16 rows x 64 B, half lines, cost three times as much here and slowed the next tile's loads).  The first
    // fragments of the next tile are in flight the whole time.
    auto finish_tile = [&](const void *out, int N, int m0, int n0) {
        const int l = opaque(lane0);
        const int r = l & 15, g_ = l >> 4;
        float sxA[TM], sxB[TM];   // row r % 8 and row 8 + r % 8 of each 16-row tile
        v4f sw4 = {1.0f, 1.0f, 1.0f, 1.0f};
        if constexpr (DEQ) {
            static_for<TM>([&](auto I) {
                sxA[decltype(I)::value] = scale_reg<C::SCL0 + 2 * decltype(I)::value>();
                sxB[decltype(I)::value] = scale_reg<C::SCL0 + 2 * decltype(I)::value + 1>();
            });
        }
        const char *const base = static_cast<const char *>(out) + ((int64_t)m0 * N + n0) * 4;
        const int64_t rows16 = (int64_t)64 * N;   // bytes from one 16-row tile to the next
        const int64_t rows8 = (int64_t)32 * N;
        const bool lo = r < 8;
        // this lane's place in a store of 8 rows x 128 B: row r % 8, and the 16 bytes 4g of column tile j (lanes
        // r < 8) or of column tile j + 1 (lanes r >= 8)
        unsigned vo = (unsigned)(((wm * 64 + (r & 7)) * N + wn * (16 * TN) + (lo ? 0 : 16) + 4 * g_) * 4);
        static_for<TN / 2>([&](auto JP) {
            constexpr int j = 2 * decltype(JP)::value;
            if constexpr (DEQ) {
                sw4[0] = scale_reg<C::SCL0 + 2 * TM + 2 * j>();
                sw4[1] = scale_reg<C::SCL0 + 2 * TM + 2 * j + 1>();
                sw4[2] = scale_reg<C::SCL0 + 2 * TM + 2 * j + 2>();
                sw4[3] = scale_reg<C::SCL0 + 2 * TM + 2 * j + 3>();
            }
            // the matrix instructions of the stage's last two groups wrote the last two column tiles a moment ago
            if constexpr (j == TN - 2) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
            static_for<TM>([&](auto I) {
                constexpr int i = decltype(I)::value;
                constexpr int r0 = vacc::ACC0 + 4 * (j * TM + i), r1 = vacc::ACC0 + 4 * ((j + 1) * TM + i);
                const char *sbase = base + i * rows16 + j * 64;
                const char *sbase8 = sbase + rows8;
                const unsigned vo_ = vo;   // (named outside the asm so that the lambda captures it)
                // vA: rows 0-7 of the pair's 16 rows: lanes r < 8 keep column tile j (their own), lanes r >= 8 take
                // column tile j + 1 from lane r - 8; vB: rows 8-15: lanes r >= 8 keep tile j + 1, lanes r < 8 take
                // tile j from lane r + 8.  One select with the rotation by eight lanes on its first source does both
                // the exchange and the choice; the accumulators are read where they live and cleared behind it.
                v4i vA, vB;
                asm volatile("s_mov_b32 vcc_lo, 0x00ff00ff\n\ts_mov_b32 vcc_hi, 0x00ff00ff\n\t"
                             "v_cndmask_b32_dpp %0, v%c12, v%c8, vcc row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
                             "v_cndmask_b32_dpp %1, v%c13, v%c9, vcc row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
                             "v_cndmask_b32_dpp %2, v%c14, v%c10, vcc row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
                             "v_cndmask_b32_dpp %3, v%c15, v%c11, vcc row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
                             "s_mov_b32 vcc_lo, 0xff00ff00\n\ts_mov_b32 vcc_hi, 0xff00ff00\n\t"
                             "v_cndmask_b32_dpp %4, v%c8, v%c12, vcc row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
                             "v_cndmask_b32_dpp %5, v%c9, v%c13, vcc row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
                             "v_cndmask_b32_dpp %6, v%c10, v%c14, vcc row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
                             "v_cndmask_b32_dpp %7, v%c11, v%c15, vcc row_ror:8 row_mask:0xf bank_mask:0xf"
                             : "=&v"(vA[0]), "=&v"(vA[1]), "=&v"(vA[2]), "=&v"(vA[3]), "=&v"(vB[0]), "=&v"(vB[1]),
                               "=&v"(vB[2]), "=&v"(vB[3])
                             : "n"(r0), "n"(r0 + 1), "n"(r0 + 2), "n"(r0 + 3), "n"(r1), "n"(r1 + 1), "n"(r1 + 2), "n"(r1 + 3)
                             : "vcc");
                if constexpr (DEQ) {
                    // rows 0-7 use the scale of row r % 8, rows 8-15 that of row 8 + r % 8 of this 16-row tile
                    v4f fA, fB;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        fA[q] = ((float)vA[q] * sxA[i]) * sw4[q];
                        fB[q] = ((float)vB[q] * sxB[i]) * sw4[q];
                    }
                    asm volatile("global_store_dwordx4 %0, %1, %2" MI_STORE_MOD "\n\ts_nop 2" ::"v"(vo_), "v"(fA), "s"(sbase) : "memory");
                    asm volatile("global_store_dwordx4 %0, %1, %2" MI_STORE_MOD "\n\ts_nop 2" ::"v"(vo_), "v"(fB), "s"(sbase8) : "memory");
                } else {
                    asm volatile("global_store_dwordx4 %0, %1, %2" MI_STORE_MOD "\n\ts_nop 2" ::"v"(vo_), "v"(vA), "s"(sbase) : "memory");
                    asm volatile("global_store_dwordx4 %0, %1, %2" MI_STORE_MOD "\n\ts_nop 2" ::"v"(vo_), "v"(vB), "s"(sbase8) : "memory");
                }
                // (the wait states behind a store: a store of more than 8 bytes reads its data registers for a few
                // cycles after it has issued, and the vector instruction behind an asm statement may already write
                // them; the compiler pads this for its own stores only.  In front of it none are needed as long as the
                // build lets no scalar be spilled: a scalar brought back by v_readlane may be read by a memory
                // instruction only five wait states later, and the compiler cannot see the asm's memory instruction.)
            });
        });
    };

    // ---- fill: stages 0 and 1 of the first tile, then its first fragments
    cursor_to((v4i){e_p, e_m0, e_n0, 0});
    nk = bt.p[e_p].K >> 7;
    {
        static_for<C::LX>([&](auto I) { issue_x(I, 0u); });
        static_for<C::LW>([&](auto I) { issue_w(I, 0u); });
        lkt = 1;
        static_for<C::LX>([&](auto I) { issue_x(I, (unsigned)XSTAGE); });
        static_for<C::LW>([&](auto I) { issue_w(I, (unsigned)WSTAGE); });
        wait_vm<C::LX + C::LW>();   // stage 0 has landed
    }
    lkt = 2;
    __syncthreads();
    // the first fragments, in the order in which every second half requests them for the next stage
    ds_read128<0>(w[0], wo0);
    static_for<TN - 1>([&](auto J1) {
        constexpr int j = decltype(J1)::value + 1;
        if constexpr (j - 1 < TM) ds_read128<(j - 1) * 2048>(xa[j - 1], xo0);
        ds_read128<j * 2048>(w[j], wo0);
    });

    for (int it = 0;; ++it) {
        // (the list is read again where the next entry is needed: it is not worth four scalar registers for a tile)
        const bool more = sload4(my + it + 1)[0] >= 0;
        bool in_cur = true;   // the cursor stands in this tile (it entered it two stages ago)
#ifdef MI_GEMM_TIMELINE
        const unsigned long long tl_a = __builtin_amdgcn_s_memtime(), tl_ra = __builtin_amdgcn_s_memrealtime();
#endif
        for (kt = 0; kt < nk; ++kt) {
            stage();
            // the cursor moves on: to the next stage of its tile, to the next tile, or off the end of the list
            if (ldv && ++lkt == lnk) {
                if (in_cur && more) cursor_to(sload4(my + it + 1));
                else ldv = false;
                in_cur = false;
            }
        }
#ifdef MI_GEMM_TIMELINE
        const unsigned long long tl_b = __builtin_amdgcn_s_memtime();
#endif
        {
            const Problem &P = bt.p[e_p];
            finish_tile(P.out, P.N, e_m0, e_n0);
        }
#ifdef MI_GEMM_TIMELINE
        {
            const unsigned long long tl_c = __builtin_amdgcn_s_memtime(), tl_rc = __builtin_amdgcn_s_memrealtime();
            if (wave == MI_TL_WAVE && opaque(lane0) == 0 && blockIdx.x < TL_WGS && it < TL_TILES) {
                unsigned long long *o = g_list_timeline + ((size_t)blockIdx.x * TL_TILES + it) * 8;
                o[0] = tl_a;    // first stage begins (ticks)
                o[1] = tl_b;    // last stage issued
                o[2] = tl_c;    // last store issued
                o[3] = tl_ra;   // real time (100 MHz) at o[0]
                o[4] = tl_rc;   // real time at o[2]
                o[5] = (unsigned long long)nk;
                o[6] = 1ull | ((unsigned long long)tl_wait1 << 8);
                o[7] = ((unsigned long long)tl_bar << 32) | tl_wait;
            }
            tl_wait = tl_bar = tl_wait1 = 0;
        }
#endif
        if (!more) break;
        first_tile = false;
        const v4i e = sload4(my + it + 1);
        e_p = e[0];
        e_m0 = e[1];
        e_n0 = e[2];
        nk = bt.p[e_p].K >> 7;
        e_sx = bt.p[e_p].sx + e_m0;
        e_sw = bt.p[e_p].sw + e_n0;
    }
}

// ---- host side: the work list

struct Tile {
    int p, m0, n0, cost;
};

// cost of a tile in K stages, plus what does not grow with K (conversion and stores, and the slower stages behind
// them: a tile of 112 stages was measured at 2.9 times a tile of 32)
static inline int tile_cost(int64_t K) { return (int)(K / 128) + 10; }

// Rounds.  The tiles of all problems, longest K first, are cut into blocks of as many tiles as an XCD has
// workgroups (problems of equal K share blocks); a block is a compact patch of a problem's tile grid, ROWS row
// tiles by slots / ROWS column tiles (4 x 8 for 32 workgroups: the patch with the fewest operand bytes per tile).
// Blocks go, longest first, to the XCD with the least work so far, and workgroup s of an XCD takes tile s of every
// block of its XCD.  All workgroups of an XCD therefore walk through the same sequence of tile lengths side by side
// and stay close to each other in K, so that one fetch into the XCD's L2 serves every workgroup that shares a row
// or a column of the patch.  Measured on the four prefill projections against a list that gave each XCD an eighth of
// every problem and balanced its workgroups tile by tile (longest tile to the least loaded workgroup): 736 MB
// instead of 1,189 MB fetched per launch (operands 256 MB), 338 against 344 us with the weights resident in the
// memory-side cache and 355 against 371 us with weights that come from HBM; patches of 1, 2 and 8 row tiles
// measured 355 / 344 / 339 us (resident) and 366 / 364 / 369 us (from HBM).
template <int BM, int BN>
static int64_t build_lists(const int64_t *mnk, int n, int cus, std::vector<v4i> *lists, int *per_wg_out)
{
    const int nx = (cus % 8 == 0) ? 8 : 1, slots = cus / nx;
    constexpr int ROWS = 4;
    std::vector<int> order((size_t)n);
    for (int p = 0; p < n; ++p) order[(size_t)p] = p;
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return mnk[3 * a + 2] > mnk[3 * b + 2]; });
    std::vector<std::vector<Tile>> blocks;
    int64_t total = 0, last_k = -1;
    for (int p : order) {
        const int64_t M = mnk[3 * p], N = mnk[3 * p + 1], K = mnk[3 * p + 2];
        const int64_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
        total += tm * tn;
        if (total > MAX_TILES) return MI_ERANGE;
        if (K != last_k) blocks.emplace_back();   // a block holds tiles of one length only
        last_k = K;
        for (int64_t rg = 0; rg < tm; rg += ROWS)
            for (int64_t col = 0; col < tn; ++col)
                for (int64_t row = rg; row < std::min<int64_t>(rg + ROWS, tm); ++row) {
                    if ((int)blocks.back().size() == slots) blocks.emplace_back();
                    Tile tl;
                    tl.p = p;
                    tl.m0 = (int)std::min<int64_t>(row * BM, M - BM);   // an edge tile moves inwards
                    tl.n0 = (int)std::min<int64_t>(col * BN, N - BN);
                    tl.cost = tile_cost(K);
                    blocks.back().push_back(tl);
                }
    }
    std::vector<std::vector<Tile>> q((size_t)cus);
    std::vector<int64_t> load((size_t)nx, 0);
    std::vector<std::vector<const std::vector<Tile> *>> mine((size_t)nx);
    for (const auto &b : blocks) {
        if (b.empty()) continue;
        int best = 0;
        for (int x = 1; x < nx; ++x)
            if (load[(size_t)x] < load[(size_t)best]) best = x;
        load[(size_t)best] += b[0].cost;
        mine[(size_t)best].push_back(&b);
    }
    for (int x = 0; x < nx; ++x) {
        // a block with fewer tiles than the XCD has workgroups runs last: the workgroups it leaves out are done,
        // instead of running ahead of their neighbours for the rest of the list
        std::stable_sort(mine[(size_t)x].begin(), mine[(size_t)x].end(),
                         [&](const std::vector<Tile> *a, const std::vector<Tile> *b) {
                             return ((int)a->size() == slots) > ((int)b->size() == slots);
                         });
        for (const auto *b : mine[(size_t)x])
            for (size_t s = 0; s < b->size(); ++s) q[s * (size_t)nx + (size_t)x].push_back((*b)[s]);   // workgroup id mod 8 = XCD
    }
    size_t longest = 0;
    for (const auto &v : q) longest = std::max(longest, v.size());
    const int per_wg = (int)longest + 1;
    if (per_wg_out) *per_wg_out = per_wg;
    if (lists) {
        lists->assign((size_t)cus * per_wg, (v4i){-1, 0, 0, 0});
        for (int w = 0; w < cus; ++w)
            for (size_t i = 0; i < q[(size_t)w].size(); ++i) {
                const Tile &tl = q[(size_t)w][i];
                (*lists)[(size_t)w * per_wg + i] = (v4i){tl.p, tl.m0, tl.n0, tl.cost};
            }
    }
    return (int64_t)cus * per_wg * (int64_t)sizeof(v4i);
}

using LC = Cfg;

static int32_t check_shapes(const int64_t *mnk, int32_t n)
{
    if (!mnk || n < 1 || n > MAX_PROBLEMS) return MI_EINVAL;
    for (int p = 0; p < n; ++p) {
        const int64_t M = mnk[3 * p], N = mnk[3 * p + 1], K = mnk[3 * p + 2];
        if (M < LC::BM || N < LC::BN || K < 128 * LC::MIN_STAGES || K % 128 || N % 16) return MI_EINVAL;
        if (M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL) return MI_ERANGE;
        if ((int64_t)127 * 127 * K > 0x7fffffffLL) return MI_ERANGE;   // int32 accumulator bound
    }
    return MI_OK;
}

}  // namespace list
}  // namespace mi

using namespace mi;

struct mi_gemm_batch {
    int32_t n;
    int32_t device;
    int32_t grid, per_wg;
    int64_t mnk[3 * list::MAX_PROBLEMS];
    const v4i *lists;   // device memory of the caller
};

extern "C" int64_t mi_gemm_batch_plan_bytes(const int64_t *mnk, int32_t n)
{
    int32_t rc = list::check_shapes(mnk, n);
    if (rc) return rc;
    return list::build_lists<list::LC::BM, list::LC::BN>(mnk, n, compute_units(), nullptr, nullptr);
}

extern "C" int64_t mi_gemm_batch_plan_host(const int64_t *mnk, int32_t n, int32_t compute_units_, int32_t *lists_out,
                                           int64_t capacity_bytes, int32_t *per_wg_out)
{
    int32_t rc = list::check_shapes(mnk, n);
    if (rc) return rc;
    if (compute_units_ < 1 || compute_units_ > 4096 || !lists_out || !per_wg_out) return MI_EINVAL;
    std::vector<v4i> lists;
    int per_wg = 0;
    const int64_t bytes = list::build_lists<list::LC::BM, list::LC::BN>(mnk, n, compute_units_, &lists, &per_wg);
    if (bytes < 0) return bytes;
    if (capacity_bytes < bytes) return MI_ENOSPC;
    memcpy(lists_out, lists.data(), (size_t)bytes);
    *per_wg_out = per_wg;
    return bytes;
}

extern "C" int32_t mi_gemm_batch_create(const int64_t *mnk, int32_t n, void *plan, int64_t plan_bytes,
                                        mi_gemm_batch **out)
{
    if (!out) return MI_EINVAL;
    *out = nullptr;
    int32_t rc = list::check_shapes(mnk, n);
    if (rc) return rc;
    if (!plan || !aligned16(plan)) return MI_EINVAL;
    std::vector<v4i> lists;
    int per_wg = 0;
    const int cus = compute_units();
    const int64_t bytes = list::build_lists<list::LC::BM, list::LC::BN>(mnk, n, cus, &lists, &per_wg);
    if (bytes < 0) return (int32_t)bytes;
    if (plan_bytes < bytes) return MI_ENOSPC;
    int dev = 0;
    MI_HIP(hipGetDevice(&dev));
    MI_HIP(hipMemcpy(plan, lists.data(), (size_t)bytes, hipMemcpyHostToDevice));   // returns when the list is in place
    mi_gemm_batch *b = new (std::nothrow) mi_gemm_batch();
    if (!b) return MI_ENOMEM;
    b->n = n;
    b->device = dev;
    b->grid = cus;
    b->per_wg = per_wg;
    for (int i = 0; i < 3 * n; ++i) b->mnk[i] = mnk[i];
    b->lists = static_cast<const v4i *>(plan);
    *out = b;
    return MI_OK;
}

extern "C" int32_t mi_gemm_batch_destroy(mi_gemm_batch *b)
{
    if (!b) return MI_EINVAL;
    delete b;
    return MI_OK;
}

template <bool DEQ>
static int32_t batch_run(mi_gemm_batch *b, const mi_gemm_problem *p, void *stream)
{
    if (!b || !p) return MI_EINVAL;
    list::Batch bt = {};
    for (int i = 0; i < b->n; ++i) {
        const mi_gemm_problem &g = p[i];
        if (g.M != b->mnk[3 * i] || g.N != b->mnk[3 * i + 1] || g.K != b->mnk[3 * i + 2]) return MI_EINVAL;
        if (!g.qx || !g.qw || !g.out || !aligned16(g.qx) || !aligned16(g.qw) || !aligned16(g.out)) return MI_EINVAL;
        if (DEQ && (!g.sx || !g.sw || !aligned4(g.sx) || !aligned4(g.sw))) return MI_EINVAL;
        list::Problem &d = bt.p[i];
        d.qx = g.qx;
        d.qw = g.qw;
        d.sx = g.sx;
        d.sw = g.sw;
        d.out = g.out;
        d.M = (int)g.M;
        d.N = (int)g.N;
        d.K = (int)g.K;
    }
    int dev = -1;
    MI_HIP(hipGetDevice(&dev));
    if (dev != b->device) return MI_EINVAL;   // the list lives in that device's memory
    MI_LDS_OPT_IN((&list::k_w8a8_list<DEQ>), list::LC::LDS);
    hipLaunchKernelGGL((list::k_w8a8_list<DEQ>), dim3((unsigned)b->grid), dim3(512), list::LC::LDS,
                       as_stream(stream), bt, b->lists, b->per_wg);
    return launch_status();
}

#ifdef MI_GEMM_TIMELINE
extern "C" __attribute__((visibility("default"))) int32_t mi_debug_gemm_list_timeline(unsigned long long *out, int32_t n, int32_t clear)
{
    if (n < 0 || n > list::TL_WGS * list::TL_TILES * 8) return MI_EINVAL;
    if (out && hipMemcpyFromSymbol(out, HIP_SYMBOL(list::g_list_timeline), (size_t)n * 8) != hipSuccess) return MI_EIO;
    if (clear) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(list::g_list_timeline)) != hipSuccess) return MI_EIO;
        if (hipMemset(p, 0, sizeof(unsigned long long) * list::TL_WGS * list::TL_TILES * 8) != hipSuccess) return MI_EIO;
    }
    return MI_OK;
}
#endif

extern "C" int32_t mi_gemm_batch_run_f32(mi_gemm_batch *b, const mi_gemm_problem *p, void *stream)
{
    return batch_run<true>(b, p, stream);
}

extern "C" int32_t mi_gemm_batch_run_i32(mi_gemm_batch *b, const mi_gemm_problem *p, void *stream)
{
    return batch_run<false>(b, p, stream);
}
