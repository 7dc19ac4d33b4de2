// Several W8A8 contractions in ONE launch: a workgroup per compute unit walks a list of output tiles.
//   acc[m,n] = sum_k qx[m,k] * qw[n,k],   y = ((float)acc * sx[m]) * sw[n]      (per problem of the batch)
//
// Why.  A prefill GEMM launched on its own spends a third of its time outside the stage loop: the gap to the
// previous kernel, the first memory round trip of 256 workgroups asking at once, and a store phase in which every
// tile of the chip writes at the same moment with the matrix pipe idle.  Its tile shape is also dictated by how
// the tile count divides by the number of compute units.  Here the tiles of all problems form one work list:
//   - one tile shape for everything (32*TM x 32*TN = 256 x 192, eight waves, two per SIMD: the stage loop of
//     gemm_pair.hip, which is the fastest one), because the list is balanced as a whole and not per problem;
//   - the first two K stages of a workgroup's next tile are requested BEFORE the current tile's sums are exchanged
//     and stored, so the next stage loop starts on data that is already in LDS;
//   - workgroups drift apart (tiles differ in K), so stores of one unit fall under the stage loops of the others.
// A tile that would cross the edge of its matrix is moved inwards until it fits: the overlap with its neighbour
// is computed twice, both times to the same values (exact integers, the same fp32 operations), so every problem
// needs only M >= 256, N >= 192; no ragged code path exists.
//
// Per wave, stage loop, LDS layout and swizzle: see gemm_pair.hip (this file repeats its stage, with the first
// stage of a tile writing the accumulators instead of adding to them).  What differs:
//   - the K halves of a wave pair meet in rounds of two accumulators (one row tile, two column tiles) through
//     2 x 8 parcels of 2 KB that lie in the third weight buffer, the only stage buffer the prefetched stages 0 and
//     1 of the next tile do not use;
//   - the epilogue's scales sit in one of two LDS areas, by tile parity (the next tile's are requested with its
//     first stages, while the current tile's are still being read).
// Memory operations complete in issue order (one counter for loads and stores), and every wait below is written
// against that order: at most 1 + 4*(LX+LW) + IH*TN = 53 are ever in flight per wave (the counter holds 63).
//
// The list itself is made on the host when the batch is created (longest tiles first, each to the least loaded
// workgroup of its XCD; tiles that run at the same time on one XCD are neighbours in column-major order, so they
// share weight columns and activation rows in that XCD's L2) and lives in device memory.
//
// Bound: int8 MFMA (2*M*N*K ops per problem).  Exact integer arithmetic.
#include <string.h>

#include <algorithm>
#include <atomic>
#include <new>
#include <vector>

#include "common.h"
#include "gemm_pair_ops.h"

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

template <int TM, int TN>
struct Cfg {
    static constexpr int BM = 32 * TM, BN = 32 * TN;
    static constexpr int NBX = 4 * TM, NBW = 4 * TN;   // 1 KB blocks (8 rows x 128 B) per stage
    static constexpr int XSTAGE = NBX * 1024, WSTAGE = NBW * 1024, XAREA = 2 * XSTAGE;
    static constexpr int STAGES = XAREA + 3 * WSTAGE;
    static constexpr int IH = TM / 2;
    static constexpr int PARCEL = 2048;                         // two accumulators of a wave
    static constexpr int PARCELS_AT = XAREA + 2 * WSTAGE;       // the third weight buffer and what follows it
    static constexpr int PARCELS = 2 * 8 * PARCEL;
    static constexpr int SCALES = (BM + BN) * 4;
    static constexpr int SCALES_AT = (STAGES > PARCELS_AT + PARCELS) ? STAGES : PARCELS_AT + PARCELS;
    static constexpr int LDS = SCALES_AT + 2 * SCALES;
    static constexpr int LX = NBX / 8, LW = NBW / 8;            // parts (pairs of loads) per loading wave and stage
    static constexpr int NS = IH * TN;                          // stores per wave and tile
    static_assert(NBX % 8 == 0 && NBW % 8 == 0, "blocks are dealt to eight waves");
    static_assert(TN % 2 == 0 && TM % 2 == 0, "the two waves of a pair finish half of the tile each");
    static_assert(TM * TN * 4 <= 192, "64 ordinary registers must remain");
    static_assert(LDS <= 160 * 1024, "LDS of a compute unit");
    static_assert(1 + 4 * (LX + LW) + NS <= 63, "the memory counter has six bits");
    static_assert(BM % 64 == 0 && BN % 64 == 0 && BM + BN <= 512, "a wave brings 64 scales of one kind");
};

// direct-to-LDS load of 4 bytes per lane: global address = sbase + voff, LDS address = ldsaddr + 4 * lane
__device__ __forceinline__ void dma4(const float *sbase, unsigned voff, unsigned ldsaddr)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                 :
                 : "v"(voff), "s"(sbase), "s"(ldsaddr)
                 : "memory", "m0");
}
#ifdef MI_GEMM_TIMELINE
// Built only into libmi355_int8_timeline.so (bench.py --gemm-timeline): wave 0 of every workgroup leaves, per tile,
// the clock ticks (s_memtime) at which the tile's first stage was in LDS, its stage loop ended and its last store
// was issued, and the 100 MHz real time at the first and the last of them.
constexpr int TL_WGS = 512, TL_TILES = 16;
__device__ unsigned long long g_list_timeline[TL_WGS * TL_TILES * 8];
#endif

__device__ __forceinline__ v4i sload4(const v4i *p)
{
    v4i v;
    asm volatile("s_load_dwordx4 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(p) : "memory");
    return v;
}

struct Epi {   // what the epilogue of a tile needs once the load side has moved on to the next tile
    void *out;
    int N, K, m0, n0;
};

// lane-derived values are recomputed in every phase of a tile from a copy of the lane number that the compiler
// cannot see through: otherwise it computes all of them once, before the tile loop, and 64 registers cannot hold them
// beside the fragments
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

template <int TM, int TN, bool DEQ>
__global__ __launch_bounds__(512) __attribute__((amdgpu_num_vgpr(vacc::ACC0 / 2))) void k_w8a8_list(
    const Batch bt, const v4i *__restrict__ lists, int per_wg)
{
    using C = Cfg<TM, TN>;
    constexpr int BM = C::BM, BN = C::BN;
    constexpr int XSTAGE = C::XSTAGE, WSTAGE = C::WSTAGE, XAREA = C::XAREA;
    constexpr int LX = C::LX, LW = C::LW, NS = C::NS, IH = C::IH;
    constexpr int R = (TN % 3 == 0) ? 3 : 4;    // weight fragment registers in rotation
    extern __shared__ __attribute__((aligned(16))) char smem[];
    // v[64 .. 255] are this kernel's accumulators, named by hand: the attribute above keeps everything the compiler
    // places below v64, and this clobber makes the wave's register count cover them
    static_assert(vacc::ACC0 + 4 * TM * TN <= 256);
    asm volatile("" ::: "v64", "v255");

    const int tid = threadIdx.x, lane0 = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int pw = wave & 3, half = wave >> 2;   // wave tile of the pair, K half of every stage
    const int wm = pw >> 1, wn = pw & 1;
    const bool loader = half == 0;               // the waves the matrix pipe serves first issue every load
    const unsigned lds_base = (unsigned)(uintptr_t)(lptr_t)smem;
    const unsigned lds_x = lds_base + pw * 1024, lds_w = lds_base + XAREA + pw * 1024;

    const v4i *const my = lists + (int64_t)blockIdx.x * per_wg;
    v4i ent = sload4(my);   // {problem or -1, first row, first column, -}
    if (ent[0] < 0) return;
    static_for<TM * TN>([&](auto I) { vacc::acc_zero4<4 * decltype(I)::value>(); });

    // ---- the tile whose stages are being loaded
    const int8_t *xtile = nullptr, *wtile = nullptr;
    unsigned voff = 0;
    int64_t bstep = 0;
    int nk = 0;

    // load side: lane l = 8*rho + c fetches the 16-byte chunk c ^ sigma of row rho of a block; wave pw fills
    // blocks pw + 4q, so one lane offset serves every block on a uniform base that moves with q
    auto lane_offset = [&](int K) {
        const int l = opaque(lane0);
        const int lrow = pw * 8 + (l >> 3);
        const unsigned lchunk = (unsigned)(((l & 7) ^ (((pw & 1) << 2) | (l >> 4))) << 4);
        return (unsigned)lrow * (unsigned)K + lchunk;
    };
    auto issue_x1 = [&](auto I, unsigned buf, int kt) {
        constexpr int p_ = decltype(I)::value;
        if constexpr (p_ < LX) {
            dma16(xtile + (int64_t)kt * 128 + (2 * p_) * bstep, voff, lds_x + buf + (2 * p_) * 4096);
            dma16(xtile + (int64_t)kt * 128 + (2 * p_ + 1) * bstep, voff, lds_x + buf + (2 * p_ + 1) * 4096);
        }
    };
    auto issue_w1 = [&](auto I, unsigned buf, int kt) {
        constexpr int p_ = decltype(I)::value;
        if constexpr (p_ < LW) {
            dma16(wtile + (int64_t)kt * 128 + (2 * p_) * bstep, voff, lds_w + buf + (2 * p_) * 4096);
            dma16(wtile + (int64_t)kt * 128 + (2 * p_ + 1) * bstep, voff, lds_w + buf + (2 * p_ + 1) * 4096);
        }
    };
    auto issue_x = [&](unsigned buf, int kt) { static_for<LX>([&](auto I) { issue_x1(I, buf, kt); }); };
    auto issue_w = [&](unsigned buf, int kt) { static_for<LW>([&](auto I) { issue_w1(I, buf, kt); }); };

    // a tile begins: its scales and its stages 0 and 1 are requested (activation buffers 0 and 1, weight buffers
    // 0 and 1: every stage buffer is free when this is called).  In the memory counter's order: scales, stage 0,
    // stage 1.  The scales go straight to their LDS area (wave w brings 64 of them: the BM row scales, then the BN
    // column scales), so that no register has to hold them while the previous tile's epilogue runs.
    auto begin_tile = [&](const v4i &e, unsigned scales_at) -> Epi {
        const Problem &P = bt.p[e[0]];
        const int K = P.K;
        nk = K >> 7;
        xtile = P.qx + (int64_t)e[1] * K;
        wtile = P.qw + (int64_t)e[2] * K;
        voff = lane_offset(K);
        bstep = (int64_t)32 * K;   // four blocks of eight rows
        if constexpr (DEQ) {
            if (wave * 64 < BM + BN) {
                const float *src = wave * 64 < BM ? P.sx + e[1] + wave * 64 : P.sw + e[2] + (wave * 64 - BM);
                dma4(src, (unsigned)opaque(lane0) * 4u, lds_base + scales_at + wave * 256);
            }
        }
        if (loader) {
            issue_x(0u, 0);
            issue_w(0u, 0);
            if (nk > 1) {
                issue_x((unsigned)XSTAGE, 1);
                issue_w((unsigned)WSTAGE, 1);
            }
        }
        Epi ep;
        ep.out = P.out;
        ep.N = P.N;
        ep.K = K;
        ep.m0 = e[1];
        ep.n0 = e[2];
        return ep;
    };

    v4i xb[TM], wa[R];
    int kt = 0;
    unsigned xo = 0, wo = 0;   // this lane's fragment addresses in activation buffer 0 / weight buffer 0
    unsigned xcur = 0, xnxt = XSTAGE, wcur = 0, wnxt = WSTAGE, wnn = 2 * WSTAGE;

    // one stage.  There is ONE copy of this code and one loop around it: a fragment register is written by an LDS
    // read the compiler cannot follow (its data arrives later), so no value of xb / wa may ever have to be moved
    // where two paths of the control flow meet.  The last stage of a tile therefore also requests "next" fragments
    // (from a buffer that holds nothing new; they are never used), and the accumulators start a tile at zero
    // (cleared by the epilogue that read them) instead of a first stage that writes them.
    auto stage = [&]() {
        const unsigned aw = add_vs(wo, wcur);
        const bool more2 = kt + 2 < nk;
        const bool ld2 = loader && more2, ld3 = loader && kt + 3 < nk;
        // Loads of a stage, one at the head of a group so that a wave never issues two in a row:
        //   group 0: weight part 2 of stage kt+2;  groups 1..LX: the activation parts of stage kt+2 (behind B1);
        //   group LX+1: weight part 3 of stage kt+2;  group TN-2 (behind B2) and TN-1: weight parts 0, 1 of stage kt+3
        static_for<TN>([&](auto J) {
            constexpr int j = decltype(J)::value;
            if constexpr (j == 0) {
                if (ld2) issue_w1(std::integral_constant<int, 2>{}, wnn, kt + 2);
            } else if constexpr (j <= LX) {
                if (ld2) issue_x1(std::integral_constant<int, j - 1>{}, xcur, kt + 2);
            } else if constexpr (j == LX + 1 && LW > 3) {
                static_assert(LW <= 4 && LX + 1 < TN - 2);
                if (ld2) issue_w1(std::integral_constant<int, 3>{}, wnn, kt + 2);
            } else if constexpr (j == TN - 1) {
                if (ld3) issue_w1(std::integral_constant<int, 1>{}, wcur, kt + 3);
            }
            if constexpr (j + 2 < TN) ds_read128<(j + 2) * 2048>(wa[(j + 2) % R], aw);
            if constexpr (j == 0) {
                // LDS returns in order: wa[0], wa[1], the activation fragments, then the read issued just now
                static_for<TM>([&](auto I) {
                    constexpr int i = decltype(I)::value;
                    wait_lgkm<TM - i>();
                    vacc::mfma_acc<4 * i>(wa[0], xb[i]);
                });
                // B1: every wave holds its activation fragments: the activation buffer is free for stage kt + 2
                __builtin_amdgcn_s_barrier();
            } else {
                if constexpr (j == TN - 2) {
                    // all reads of the current weight buffer have been issued: drain them and, in a loading wave,
                    // its share of the next stage (memory operations complete in order: the loads of later stages
                    // may stay in flight; whatever this wave stored for its previous tile lies before them)
                    if (loader) {
                        if (more2) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(2 * (LX + LW)) : "memory");
                        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                    } else {
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    }
                    __builtin_amdgcn_s_barrier();   // B2: stage kt+1 is visible, the weight buffer of stage kt is free
                    if (ld3) issue_w1(std::integral_constant<int, 0>{}, wcur, kt + 3);
                } else if constexpr (j < TN - 2) {
                    wait_lgkm<2>();   // wa[j] is in; wa[j+1] and the read issued just now may stay in flight
                }
                if constexpr (j == TN - 1) {
                    const unsigned nax = add_vs(xo, xnxt);
                    static_for<TM>([&](auto I) {
                        constexpr int i = decltype(I)::value;
                        vacc::mfma_acc<4 * (j * TM + i)>(wa[j % R], xb[i]);
                        ds_read128<i * 2048>(xb[i], nax);   // xb[i] has been read
                    });
                } else {
                    static_for<TM>([&](auto I) {
                        constexpr int i = decltype(I)::value;
                        vacc::mfma_acc<4 * (j * TM + i)>(wa[j % R], xb[i]);
                    });
                }
                if constexpr (j == TN - 2) {   // wa[0] and wa[1] were last read by groups before this one
                    const unsigned naw = add_vs(wo, wnxt);
                    ds_read128<0>(wa[0], naw);
                    ds_read128<2048>(wa[1], naw);
                }
            }
        });
        {
            const unsigned t = xcur; xcur = xnxt; xnxt = t;
            const unsigned u = wcur; wcur = wnxt; wnxt = wnn; wnn = u;
        }
    };
    static_assert(LW >= 3 && (TN - 1) % R >= 2 && (TN - 2) % R != 0 && LX <= TN - 2,
                  "the last group must not use wa[0] or wa[1], nor the one before it wa[0]");

    // ---- the two partial sums of a wave tile meet.  Wave `half` finishes row tiles i in [half*IH, +IH) of every
    // column tile; a round hands one row tile of two neighbouring column tiles to the partner (2 KB, two parcel
    // areas in turn: one barrier a round), adds the partner's parcel to its own accumulators and stores the pair:
    // 8 rows x 128 B per store instruction.  Both forms are compiled and a scalar branch picks one, so that every
    // accumulator register is named by a constant.
    auto finish = [&](auto HALF, const Epi &e, unsigned scales_at) {
        constexpr int hf = decltype(HALF)::value;
        constexpr int NR = IH * (TN / 2);   // rounds
        const int l = opaque(lane0);
        const int r = l & 15, g_ = l >> 4;
        const bool lo = r < 8;
        const float *const s_sx = reinterpret_cast<const float *>(smem + scales_at);
        const float *const s_sw = s_sx + BM;
        float *const y = static_cast<float *>(e.out);
        int32_t *const acc_out = static_cast<int32_t *>(e.out);
        const int N = e.N;
        const unsigned mine = lds_base + C::PARCELS_AT + wave * C::PARCEL + l * 16;
        const unsigned theirs = lds_base + C::PARCELS_AT + (wave ^ 4) * C::PARCEL + l * 16;
        const int ncol = e.n0 + wn * TN * 16 + (lo ? 0 : 16) + 4 * g_;
        float4 sw4[TN / 2];
#pragma unroll
        for (int rd = 0; rd < TN / 2; ++rd) {
            sw4[rd] = float4{1.0f, 1.0f, 1.0f, 1.0f};
            if constexpr (DEQ) sw4[rd] = *reinterpret_cast<const float4 *>(s_sw + (wn * TN + 2 * rd) * 16 + (lo ? 0 : 16) + 4 * g_);
        }
        // round rnd = ii * (TN/2) + rd: row tile ii of this wave's half, column tiles 2rd and 2rd+1
        auto hand_over = [&](auto RND) {
            constexpr int rnd = decltype(RND)::value;
            if constexpr (rnd < NR) {
                constexpr int ii = rnd / (TN / 2), rd = rnd % (TN / 2);
                constexpr int ip = (1 - hf) * IH + ii;
                constexpr int area = (rnd & 1) * 8 * C::PARCEL;
                vacc::acc_to_lds<4 * ((2 * rd) * TM + ip), area>(mine);
                vacc::acc_to_lds<4 * ((2 * rd + 1) * TM + ip), area + 1024>(mine);
            }
        };
        hand_over(std::integral_constant<int, 0>{});
        static_for<NR>([&](auto RND) {
            constexpr int rnd = decltype(RND)::value;
            constexpr int ii = rnd / (TN / 2), rd = rnd % (TN / 2);
            constexpr int i = hf * IH + ii, ip = (1 - hf) * IH + ii;
            constexpr int area = (rnd & 1) * 8 * C::PARCEL;
            // the parcels of this round are in LDS (the compiler does not count the asm's LDS writes), and every
            // wave has read what it wanted from the round before the last: the other area is free again
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            v4i o0, o1;
            ds_read128<area>(o0, theirs);
            ds_read128<area + 1024>(o1, theirs);
            hand_over(std::integral_constant<int, rnd + 1>{});   // under the latency of the reads above
            float sxA = 1.0f, sxB = 1.0f;
            if constexpr (DEQ) {
                const float *tsx = s_sx + (wm * TM + i) * 16;
                sxA = tsx[r & 7];
                sxB = tsx[8 + (r & 7)];
            }
            const int mA = e.m0 + (wm * TM + i) * 16 + (r & 7);
            const int64_t at = (int64_t)mA * N + ncol + rd * 32;
            asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(rnd + 1 < NR ? 2 : 0) : "memory");   // o0, o1 are in
            const v4i a0 = vacc::acc_plus<4 * ((2 * rd) * TM + i)>(o0);
            const v4i a1 = vacc::acc_plus<4 * ((2 * rd + 1) * TM + i)>(o1);
            v4i t0, t1;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                t0[q] = ror8(a0[q]);
                t1[q] = ror8(a1[q]);
            }
            const v4i vA = lo ? a0 : t1;  // rows 0-7:  lanes r<8 tile 2rd (own), lanes r>=8 tile 2rd+1 (from lane r-8)
            const v4i vB = lo ? t0 : a1;  // rows 8-15: lanes r>=8 tile 2rd+1 (own), lanes r<8 tile 2rd (from lane r+8)
            store4<DEQ>(y, acc_out, at, vA, sxA, sw4[rd]);
            store4<DEQ>(y, acc_out, at + (int64_t)8 * N, vB, sxB, sw4[rd]);
            // the two accumulators of this wave's own row tile have been read: they start the next tile at zero
            // (the two that were handed over are cleared once their LDS writes are known to be done: next round)
            vacc::acc_zero4<4 * ((2 * rd) * TM + i)>();
            vacc::acc_zero4<4 * ((2 * rd + 1) * TM + i)>();
        });
        // every LDS write of the hand-overs has completed (each round waited for the previous ones)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        static_for<IH * TN>([&](auto Q) {
            constexpr int q = decltype(Q)::value;
            constexpr int j = q / IH, ii = q % IH;
            vacc::acc_zero4<4 * (j * TM + (1 - hf) * IH + ii)>();
        });
    };

    Epi ce = begin_tile(ent, (unsigned)C::SCALES_AT);
    bool first = true;
    for (int it = 0;; ++it) {
        const unsigned scales_at = (unsigned)(C::SCALES_AT + (it & 1) * C::SCALES);
        // ---- stage 0 (and the scales before it) have landed when at most stage 1 and, behind it, the stores of
        // the previous tile are still in flight
        if (loader) {
            if (first) {
                if (nk > 1) wait_vm<2 * (LX + LW)>();
                else wait_vm<0>();
            } else {
                if (nk > 1) wait_vm<2 * (LX + LW) + NS>();
                else wait_vm<NS>();
            }
        } else {
            if (first) wait_vm<0>();
            else wait_vm<NS>();
        }
        __syncthreads();   // also: every wave has left the previous tile's last exchange round (third weight buffer)
#ifdef MI_GEMM_TIMELINE
        const unsigned long long tl_a = __builtin_amdgcn_s_memtime(), tl_ra = __builtin_amdgcn_s_memrealtime();
#endif
        xcur = 0; xnxt = XSTAGE; wcur = 0; wnxt = WSTAGE; wnn = 2 * WSTAGE;
        voff = lane_offset(ce.K);
        if (loader && nk > 2) {   // the first two parts of stage 2; stage 0 issues the rest (as stage kt does for kt + 2)
            issue_w1(std::integral_constant<int, 0>{}, wnn, 2);
            issue_w1(std::integral_constant<int, 1>{}, wnn, 2);
        }
        {   // read side: fragment (16 rows, this wave's K half): lane (r = l%16, g = l/16) reads row r, chunk 4*half + g
            const int l = opaque(lane0);
            const int r = l & 15, g_ = l >> 4;
            const int rho = r & 7, bpar = r >> 3;
            const int sigma = (bpar << 2) | (rho >> 1);
            const unsigned roff = bpar * 1024 + ((8 * rho + ((4 * half + g_) ^ sigma)) << 4);
            xo = lds_base + wm * TM * 2048 + roff;
            wo = lds_base + XAREA + wn * TN * 2048 + roff;
        }
        {   // first fragments of stage 0, in the order every later stage requests them
            ds_read128<0>(wa[0], wo);
            ds_read128<2048>(wa[1], wo);
            static_for<TM>([&](auto I) { ds_read128<decltype(I)::value * 2048>(xb[decltype(I)::value], xo); });
        }
#ifdef MI_GEMM_TIMELINE
        const int nk_done = nk;
#endif
        for (kt = 0; kt < nk; ++kt) stage();
        // everything of this wave is home; 2 x 16 wait states cover the longest MFMA-result -> read hazard
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\ns_nop 15\ns_nop 15" ::: "memory");
        __syncthreads();   // every wave is done with the stage buffers
#ifdef MI_GEMM_TIMELINE
        const unsigned long long tl_b = __builtin_amdgcn_s_memtime();
#endif

        // ---- the next tile's first stages go out, then this tile's sums meet and leave
        ent = sload4(my + it + 1);
        const bool more = ent[0] >= 0;
        Epi ne = ce;
        if (more) ne = begin_tile(ent, (unsigned)(C::SCALES_AT + ((it + 1) & 1) * C::SCALES));
#ifdef MI_GEMM_TIMELINE
        const unsigned long long tl_b2 = __builtin_amdgcn_s_memtime();
#endif
        if (half == 0) finish(std::integral_constant<int, 0>{}, ce, scales_at);
        else finish(std::integral_constant<int, 1>{}, ce, scales_at);
#ifdef MI_GEMM_TIMELINE
        {
            const unsigned long long tl_c = __builtin_amdgcn_s_memtime(), tl_rc = __builtin_amdgcn_s_memrealtime();
            if (wave == 0 && opaque(lane0) == 0 && blockIdx.x < TL_WGS && it < TL_TILES) {
                unsigned long long *o = g_list_timeline + ((size_t)blockIdx.x * TL_TILES + it) * 8;
                o[0] = tl_a;    // first stage in LDS (ticks)
                o[1] = tl_b;    // stage loop done
                o[2] = tl_c;    // last store issued, next tile's first stages requested
                o[3] = tl_ra;   // real time (100 MHz) at o[0]
                o[4] = tl_rc;   // real time at o[2]
                o[5] = (unsigned long long)nk_done;
                o[6] = 1;
                o[7] = tl_b2;   // next tile's first stages requested
            }
        }
#endif
        if (!more) break;
        ce = ne;
        first = false;
    }
}

// ---- host side: the work list

struct Tile {
    int p, m0, n0, cost;
};

// cost of a tile in K stages: its stage loop plus the exchange and stores
static inline int tile_cost(int64_t K) { return (int)(K / 128) + 4; }

template <int BM, int BN>
static int64_t build_lists(const int64_t *mnk, int n, int cus, std::vector<v4i> *lists, int *per_wg_out)
{
    const int nx = (cus % 8 == 0) ? 8 : 1, slots = cus / nx;
    std::vector<std::vector<Tile>> per_xcd((size_t)nx);
    int64_t total = 0;
    for (int p = 0; p < n; ++p) {
        const int64_t M = mnk[3 * p], N = mnk[3 * p + 1], K = mnk[3 * p + 2];
        const int64_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN, nt = tm * tn;
        total += nt;
        if (total > MAX_TILES) return MI_ERANGE;
        for (int64_t t = 0; t < nt; ++t) {   // column-major: the row tiles of one weight column are neighbours
            const int64_t col = t / tm, row = t % tm;
            const int x = (int)((t * nx / nt + p) % nx);
            Tile tl;
            tl.p = p;
            tl.m0 = (int)std::min<int64_t>(row * BM, M - BM);   // an edge tile moves inwards
            tl.n0 = (int)std::min<int64_t>(col * BN, N - BN);
            tl.cost = tile_cost(K);
            per_xcd[(size_t)x].push_back(tl);
        }
    }
    std::vector<std::vector<Tile>> q((size_t)cus);
    for (int x = 0; x < nx; ++x) {
        auto &v = per_xcd[(size_t)x];
        std::stable_sort(v.begin(), v.end(), [](const Tile &a, const Tile &b) { return a.cost > b.cost; });
        std::vector<int64_t> load((size_t)slots, 0);
        for (const Tile &tl : v) {
            int best = 0;
            for (int s = 1; s < slots; ++s)
                if (load[(size_t)s] < load[(size_t)best]) best = s;
            load[(size_t)best] += tl.cost;
            q[(size_t)(best * nx + x)].push_back(tl);   // workgroup id mod 8 = XCD
        }
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

constexpr int TM_ = 8, TN_ = 6;
using LC = Cfg<TM_, TN_>;

static int32_t check_shapes(const int64_t *mnk, int32_t n)
{
    if (!mnk || n < 1 || n > MAX_PROBLEMS) return MI_EINVAL;
    for (int p = 0; p < n; ++p) {
        const int64_t M = mnk[3 * p], N = mnk[3 * p + 1], K = mnk[3 * p + 2];
        if (M < LC::BM || N < LC::BN || K < 128 || K % 128 || N % 16) return MI_EINVAL;
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
    std::atomic<bool> attr_set[2];
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
    b->attr_set[0] = b->attr_set[1] = false;
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
    const void *fn = reinterpret_cast<const void *>(&list::k_w8a8_list<list::TM_, list::TN_, DEQ>);
    if (!b->attr_set[DEQ].load(std::memory_order_acquire)) {
        MI_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, list::LC::LDS));
        b->attr_set[DEQ].store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL((list::k_w8a8_list<list::TM_, list::TN_, DEQ>), dim3((unsigned)b->grid), dim3(512), list::LC::LDS,
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
