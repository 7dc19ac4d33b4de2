// W8A8 contraction for prefill, eight waves per workgroup: two waves on every SIMD.
//   acc[m,n] = sum_k qx[m,k] * qw[n,k],   y = ((float)acc * sx[m]) * sw[n]
//
// Why a second form of the tiled kernel.  With one wave per SIMD every cycle in which the wave issues something
// else (a direct-to-LDS load holds its issue slot for some 40 cycles), waits for a fragment or stands at a barrier
// is a cycle in which no matrix instruction starts.  Here a SIMD holds two waves, and while one of them does any
// of that, the other feeds the matrix pipe.
//
// A wave then owns 256 registers instead of 512, so the two waves of a SIMD share ONE wave tile of the four-wave
// kernel (16*TM x 16*TN outputs, TM*TN accumulators of four registers) and split every 128-byte K stage between
// them: wave p (0..3) takes the first 64 bytes of each stage, wave p + 4 the second.  LDS layout, swizzle, load
// shapes and bytes read from LDS per matrix instruction are those of the four-wave kernel; each wave issues half
// of the stage's matrix instructions, and the two partial sums of a tile meet in LDS after the last stage (each wave
// then finishes half of the row tiles).
// The matrix pipe serves the lower-numbered wave of a SIMD first, so waves 0..3 run ahead of their partners and
// would spend the difference at the barriers: they issue ALL loads of a stage, their partners none.
//
// Registers.  TM*TN*4 accumulators (192 at 8 x 6) leave 64 ordinary registers, too few for the compiler to be
// trusted with the accumulators as well: they are numbered by hand (a0 .. a(4*TM*TN-1), accumulator (j, i) at
// 4*(j*TM+i)), written only by asm, and the compiler, which sees them as clobbered, keeps everything else in the
// ordinary registers.  The matrix instructions are asm, so the hazards the compiler would pad are padded by hand:
// no operand of theirs is written by the vector ALU (fragments come from LDS reads, the accumulators are cleared
// once, wait states behind), and the epilogue reads the accumulators only after the longest result latency.
//
// Stage loop (per wave; stage s lives in activation buffer s % 2 and weight buffer s % 3; TN groups of TM matrix
// instructions, group j = weight fragment j against the TM activation fragments):
//   group 0 takes the activation fragments as they arrive, then barrier B1: every wave holds its activation
//   fragments, the activation buffer is free for the loads of stage s+2;
//   weight fragments are read two groups ahead into a ring of registers;
//   before group TN-2: the loads of stage s+1 have landed, barrier B2 -> stage s+1 is visible and the weight buffer
//   of stage s is free for stage s+3;
//   behind group TN-2 the first two weight fragments of stage s+1 are requested, and in group TN-1 each activation
//   fragment of stage s+1 right behind the last instruction that reads the old one.
//
// Whole tiles only (M a multiple of 32*TM, N of 32*TN): ragged shapes stay with the four-wave kernel.
//
// Bound: int8 MFMA (2*M*N*K ops).  Exact integer arithmetic.
#include <utility>

#include "common.h"
#include "gemm_pair_ops.h"

namespace mi {

namespace pair {

struct Grid {
    int tiles_m, tiles_n;
    int pm, pn;  // XCD partition; pm == 0 -> plain row-major tile order
};


#ifdef MI_GEMM_TIMELINE
// Built only into libmi355_int8_timeline.so (bench.py --gemm-timeline): waves 0 and 4 of every workgroup leave the
// clock ticks (s_memtime) of the kernel's three phases and the 100 MHz real time of entry and end.  Five clock reads
// a wave; the stage loop itself is untouched.
constexpr int TIMELINE_WGS = 4096;
__device__ unsigned long long g_timeline[TIMELINE_WGS * 2 * 8];
#endif

template <int TM, int TN>
struct Cfg {
    static constexpr int NBX = 4 * TM, NBW = 4 * TN;   // 1 KB blocks (8 rows x 128 B) per stage
    static constexpr int NWB = (2 * NBX + 3 * NBW + 4 <= 160) ? 3 : 2;
    static constexpr int STAGES = (2 * NBX + NWB * NBW) * 1024;
    static constexpr int SCALES = (32 * TM + 32 * TN) * 4;   // the epilogue's scales wait in LDS
    static constexpr int LDS = STAGES + SCALES;
    static_assert(NBX % 8 == 0 && NBW % 8 == 0, "blocks are dealt to eight waves");
    static_assert(TN % 2 == 0, "the two waves of a pair finish half of the column tiles each");
    static_assert(TM * TN * 4 <= 192, "64 ordinary registers must remain");
};

template <int TM, int TN, bool DEQ>
__global__ __launch_bounds__(512) void k_w8a8_pair(const int8_t *__restrict__ qx, const int8_t *__restrict__ qw,
                                                   const float *__restrict__ sx, const float *__restrict__ sw,
                                                   int32_t *__restrict__ acc_out, float *__restrict__ y, int M,
                                                   int N, int K, Grid gg)
{
    using C = Cfg<TM, TN>;
    constexpr int BM = 32 * TM, BN = 32 * TN;
    constexpr int NBX = C::NBX, NBW = C::NBW, NWB = C::NWB;
    constexpr int XSTAGE = NBX * 1024, WSTAGE = NBW * 1024, XAREA = 2 * XSTAGE;
    constexpr int LX = NBX / 8, LW = NBW / 8;   // loads per wave and stage
    constexpr int R = (TN % 3 == 0) ? 3 : 4;    // weight fragment registers in rotation
    extern __shared__ __attribute__((aligned(16))) char smem[];
    // the accumulation registers are this kernel's own: the compiler only has to know that they are in use
    asm volatile("" ::: "a0", "a31", "a63", "a95", "a127", "a159", "a191");

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int pw = wave & 3, half = wave >> 2;   // wave tile of the pair, K half of every stage
#ifdef MI_GEMM_TIMELINE
    const unsigned long long tl_entry = __builtin_amdgcn_s_memtime(), tl_rentry = __builtin_amdgcn_s_memrealtime();
#endif

    int tile_m, tile_n;
    {
        const int w = blockIdx.x;
        if (gg.pm) {
            const int x = w & 7, li = w >> 3;
            const int sub_m = gg.tiles_m / gg.pm, sub_n = gg.tiles_n / gg.pn;
            tile_m = (x / gg.pn) * sub_m + li / sub_n;
            tile_n = (x % gg.pn) * sub_n + li % sub_n;
        } else {
            tile_m = w / gg.tiles_n;
            tile_n = w % gg.tiles_n;
        }
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    // load side.  The waves of K half 0 issue all loads of a stage (they run ahead of their partners, which the
    // matrix pipe serves second, and would otherwise wait at the barriers): wave pw fills blocks b = pw + 4q of
    // each stage; lane l = 8*rho + c fetches the 16-byte chunk c ^ sigma of row rho of the block.  b % 2 = pw % 2,
    // so one 32-bit lane offset serves every block of both operands, on a uniform 64-bit base that moves with q.
    unsigned voff;
    {
        const int rho = lane >> 3, c = lane & 7;
        const int sigma = ((pw & 1) << 2) | (rho >> 1);
        voff = (unsigned)(pw * 8 + rho) * (unsigned)K + (unsigned)((c ^ sigma) << 4);
    }
    const bool loader = half == 0;
    const int64_t bstep = (int64_t)32 * K;   // four blocks of eight rows
    const int8_t *const xtile = qx + (int64_t)m0 * K;
    const int8_t *const wtile = qw + (int64_t)n0 * K;
    const unsigned lds_base = (unsigned)(uintptr_t)(lptr_t)smem;
    const unsigned lds_x = lds_base + pw * 1024, lds_w = lds_base + XAREA + pw * 1024;
    // part p of a stage's loads = blocks q = 2p, 2p + 1 of this wave (LX parts of activations, LW of weights)
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

    // read side: fragment (16 rows, this wave's K half): lane (r = l%16, g = l/16) reads row r, chunk 4*half + g
    const int r = lane & 15, g_ = lane >> 4;
    const int wm = pw >> 1, wn = pw & 1;
    unsigned roff;
    {
        const int rho = r & 7, bpar = r >> 3;
        const int sigma = (bpar << 2) | (rho >> 1);
        roff = bpar * 1024 + ((8 * rho + ((4 * half + g_) ^ sigma)) << 4);
    }
    const unsigned xo = lds_base + wm * TM * 2048 + roff, wo = lds_base + XAREA + wn * TN * 2048 + roff;


    // the scales of the epilogue: requested now, parked in LDS behind the stage buffers once the first stage has
    // landed (they precede it in the in-order memory counter), read back after the last stage
    float *const s_sx = reinterpret_cast<float *>(smem + C::STAGES);   // [BM]
    float *const s_sw = s_sx + BM;                                     // [BN]
    float stage_scale = 0.0f;
    if constexpr (DEQ) {
        const float *base = tid < BM ? sx : sw;
        const int idx = tid < BM ? m0 + tid : n0 + tid - BM;
        if (tid < BM + BN) {
            const float *p = base + idx;
            asm volatile("global_load_dword %0, %1, off" : "=v"(stage_scale) : "v"(p) : "memory");
        }
    }

    const int nk = K >> 7;
    unsigned xcur = 0, xnxt = XSTAGE;
    unsigned wcur = 0, wnxt = WSTAGE, wnn = (NWB == 3) ? 2 * WSTAGE : 0;
    if (loader) {
        issue_x(0u, 0);
        issue_w(0u, 0);
        if (nk > 1) {
            issue_x(xnxt, 1);
            issue_w(wnxt, 1);
        }
        if (nk > 2) {   // the first two parts of stage 2; stage 0 issues the rest (as every stage kt does for kt + 2)
            issue_w1(std::integral_constant<int, 0>{}, wnn, 2);
            issue_w1(std::integral_constant<int, 1>{}, wnn, 2);
        }
    }
    // cleared while the first loads are on their way
    static_for<4 * TM * TN>([&](auto I) { acc_zero<decltype(I)::value>(); });
    // stage 0 (and the scales before it) have landed when at most the later loads are still in flight
    // (a wave that loads nothing has only its scale on the way)
    if (!loader) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (nk > 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (LX + LW + 2)) : "memory");
    else if (nk > 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (LX + LW)) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (DEQ) {
        static_assert(BM + BN <= 512, "one scale per thread");
        if (tid < BM + BN) s_sx[tid] = stage_scale;   // s_sw follows s_sx
    }
    __syncthreads();

    v4i xb[TM], wa[R];
    {   // first fragments of stage 0, in the order every later stage requests them
        ds_read128<0>(wa[0], wo);
        ds_read128<2048>(wa[1], wo);
        static_for<TM>([&](auto I) { ds_read128<decltype(I)::value * 2048>(xb[decltype(I)::value], xo); });
    }
    int kt = 0;
#ifdef MI_GEMM_TIMELINE
    const unsigned long long tl_loop0 = __builtin_amdgcn_s_memtime();
#endif
    // one stage; LAST: no stage follows, nothing is requested
    auto stage = [&](auto LAST_) {
        constexpr bool LAST = decltype(LAST_)::value;
        const unsigned aw = wo + wcur;
        const unsigned nax = xo + xnxt, naw = wo + wnxt;
        const bool more2 = kt + 2 < nk;
        const bool ld2 = loader && more2, ld3 = loader && kt + 3 < nk;
        // Loads of a stage, one at the head of a group so that a wave never issues two in a row (each holds the
        // wave's issue slot for some 40 cycles, in which its SIMD has only the other wave's matrix instructions):
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
                    mfma_acc<4 * i>(wa[0], xb[i]);
                });
                // B1: every wave holds its activation fragments: the activation buffer is free for stage kt + 2
                __builtin_amdgcn_s_barrier();
            } else {
                if constexpr (j == TN - 2) {
                    // all reads of the current weight buffer have been issued: drain them and this wave's share
                    // of the next stage (loads return in order: those of later stages may stay in flight)
                    if (more2) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(2 * (LX + LW)) : "memory");
                    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                    __builtin_amdgcn_s_barrier();   // B2: stage kt+1 is visible, the weight buffer of stage kt is free
                    if (ld3) issue_w1(std::integral_constant<int, 0>{}, wcur, kt + 3);
                } else if constexpr (j < TN - 2) {
                    wait_lgkm<2>();   // wa[j] is in; wa[j+1] and the read issued just now may stay in flight
                }
                static_for<TM>([&](auto I) {
                    constexpr int i = decltype(I)::value;
                    mfma_acc<4 * (j * TM + i)>(wa[j % R], xb[i]);
                    if constexpr (j == TN - 1 && !LAST) ds_read128<i * 2048>(xb[i], nax);   // xb[i] has been read
                });
                if constexpr (j == TN - 2 && !LAST) {   // wa[0] and wa[1] were last read by groups before this one
                    ds_read128<0>(wa[0], naw);
                    ds_read128<2048>(wa[1], naw);
                }
            }
        });
        {
            const unsigned t = xcur; xcur = xnxt; xnxt = t;
            if constexpr (NWB == 3) { const unsigned u = wcur; wcur = wnxt; wnxt = wnn; wnn = u; }
            else { const unsigned u = wcur; wcur = wnxt; wnxt = u; }
        }
    };
    static_assert(NWB == 3 && LW >= 3 && (TN - 1) % R >= 2 && (TN - 2) % R != 0 && LX <= TN - 2,
                  "the last group must not use wa[0] or wa[1], nor the one before it wa[0]");
    for (; kt + 1 < nk; ++kt) stage(std::false_type{});
    stage(std::true_type{});
#ifdef MI_GEMM_TIMELINE
    const unsigned long long tl_loop1 = __builtin_amdgcn_s_memtime();
#endif
    // everything of this wave is home; 2 x 16 wait states cover the longest MFMA-result -> read hazard
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\ns_nop 15\ns_nop 15" ::: "memory");
    __syncthreads();   // every wave is done with the stage buffers: they carry the exchange below

    // ---- the two partial sums of a wave tile meet.  Wave `half` finishes row tiles i in [half*TM/2, +TM/2) of every
    // column tile; it hands the other row tiles of its accumulators to its partner through LDS, one pair of column
    // tiles a round (2 * TM/2 KB a wave; two parcel areas in turn, so one barrier a round), adds the partner's
    // parcel to its own and stores the pair: 8 rows x 128 B per store instruction.
    constexpr int IH = TM / 2;
    constexpr int PARCEL = 2 * IH * 1024;
    static_assert(2 * 8 * PARCEL <= C::STAGES, "two parcel areas fit the stage buffers");
    const bool lo = r < 8;

    // `half` is uniform over the wave: both forms of the exchange are compiled and a scalar branch picks one, so
    // that every accumulator register is named by a constant
    auto finish = [&](auto HALF) {
        constexpr int hf = decltype(HALF)::value;
        float sxA[IH], sxB[IH];
#pragma unroll
        for (int ii = 0; ii < IH; ++ii) {
            sxA[ii] = sxB[ii] = 1.0f;
            if constexpr (DEQ) {
                const float *tsx = s_sx + (wm * TM + hf * IH + ii) * 16;
                sxA[ii] = tsx[r & 7];
                sxB[ii] = tsx[8 + (r & 7)];
            }
        }
        static_for<TN / 2>([&](auto RD) {
            constexpr int rd = decltype(RD)::value;
            char *const mine = smem + ((rd & 1) * 8 + wave) * PARCEL;
            const char *const theirs = smem + ((rd & 1) * 8 + (wave ^ 4)) * PARCEL;
            // hand over: column tiles 2rd, 2rd+1, the partner's row tiles
            static_for<2>([&](auto JJ) {
                static_for<IH>([&](auto II) {
                    constexpr int jj = decltype(JJ)::value, ii = decltype(II)::value;
                    constexpr int i = (1 - hf) * IH + ii, j = 2 * rd + jj;
                    *reinterpret_cast<v4i *>(mine + (jj * IH + ii) * 1024 + lane * 16) = acc_read4<4 * (j * TM + i)>();
                });
            });
            __syncthreads();
            float4 sw4 = {1.0f, 1.0f, 1.0f, 1.0f};
            if constexpr (DEQ) sw4 = *reinterpret_cast<const float4 *>(s_sw + (wn * TN + 2 * rd) * 16 + (lo ? 0 : 16) + 4 * g_);
            const int n = n0 + (wn * TN + 2 * rd) * 16 + (lo ? 0 : 16) + 4 * g_;
            // take over, add, store
            static_for<IH>([&](auto II) {
                constexpr int ii = decltype(II)::value;
                constexpr int i = hf * IH + ii;
                const int mrow = m0 + (wm * TM + i) * 16;
                const int mA = mrow + (r & 7), mB = mrow + 8 + (r & 7);
                const v4i a0 = acc_read4<4 * ((2 * rd) * TM + i)>() +
                               *reinterpret_cast<const v4i *>(theirs + (0 * IH + ii) * 1024 + lane * 16);
                const v4i a1 = acc_read4<4 * ((2 * rd + 1) * TM + i)>() +
                               *reinterpret_cast<const v4i *>(theirs + (1 * IH + ii) * 1024 + lane * 16);
                v4i t0, t1;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    t0[e] = ror8(a0[e]);
                    t1[e] = ror8(a1[e]);
                }
                const v4i vA = lo ? a0 : t1;  // rows 0-7:  lanes r<8 tile 2rd (own), lanes r>=8 tile 2rd+1 (from lane r-8)
                const v4i vB = lo ? t0 : a1;  // rows 8-15: lanes r>=8 tile 2rd+1 (own), lanes r<8 tile 2rd (from lane r+8)
                store4<DEQ>(y, acc_out, (int64_t)mA * N + n, vA, sxA[ii], sw4);
                store4<DEQ>(y, acc_out, (int64_t)mB * N + n, vB, sxB[ii], sw4);
            });
        });
    };
    // whole tiles only (the launcher sends ragged shapes to the four-wave kernel)
    if (half == 0) finish(std::integral_constant<int, 0>{});
    else finish(std::integral_constant<int, 1>{});
#ifdef MI_GEMM_TIMELINE
    {
        const unsigned long long tl_issued = __builtin_amdgcn_s_memtime();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const unsigned long long tl_done = __builtin_amdgcn_s_memtime(), tl_rdone = __builtin_amdgcn_s_memrealtime();
        if (lane == 0 && pw == 0 && blockIdx.x < TIMELINE_WGS) {
            unsigned long long *o = g_timeline + (blockIdx.x * 2 + half) * 8;
            o[0] = tl_loop0 - tl_entry;    // first instruction -> first stage in LDS, first fragments requested
            o[1] = tl_loop1 - tl_loop0;    // the stage loop
            o[2] = tl_issued - tl_loop1;   // exchange of the K halves and the stores, to the last store issued
            o[3] = tl_done - tl_issued;    // this wave's stores acknowledged
            o[4] = tl_done - tl_entry;
            o[5] = tl_rdone - tl_rentry;
            o[6] = tl_rentry;
            o[7] = tl_rdone;
        }
    }
#endif
}

template <int TM, int TN, bool DEQ>
static int32_t launch(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc, float *y, int M,
                      int N, int K, hipStream_t s)
{
    constexpr int BM = 32 * TM, BN = 32 * TN;
    constexpr int LDS = Cfg<TM, TN>::LDS;
    // the kernel has no bounds checks: its direct-to-LDS loads and its stores address whole tiles and whole stages
    if (M <= 0 || N <= 0 || M % BM != 0 || N % BN != 0 || K < 128 || K % 128 != 0) return MI_EINVAL;
    MI_LDS_OPT_IN((&k_w8a8_pair<TM, TN, DEQ>), LDS);
    Grid gg;
    gg.tiles_m = (M + BM - 1) / BM;
    gg.tiles_n = (N + BN - 1) / BN;
    gg.pm = gg.pn = 0;
    // choose the 8-way partition that gives each XCD the fewest distinct rows + columns
    int64_t best = -1;
    const int cand[4][2] = {{1, 8}, {2, 4}, {4, 2}, {8, 1}};
    for (int c = 0; c < 4; ++c) {
        const int pm = cand[c][0], pn = cand[c][1];
        if (gg.tiles_m % pm || gg.tiles_n % pn) continue;
        const int64_t bytes = (int64_t)(gg.tiles_m / pm) * BM + (int64_t)(gg.tiles_n / pn) * BN;
        if (best < 0 || bytes < best) { best = bytes; gg.pm = pm; gg.pn = pn; }
    }
    const dim3 grid((unsigned)(gg.tiles_m * gg.tiles_n)), blk(512);
    hipLaunchKernelGGL((k_w8a8_pair<TM, TN, DEQ>), grid, blk, LDS, s, qx, qw, sx, sw, acc, y, M, N, K, gg);
    return launch_status();
}

}  // namespace pair

// the eight-wave form of the (tm, tn) wave tile: compiled for (8, 6) and (4, 8) only
template <bool DEQ>
int32_t launch_pair(int tm, int tn, const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc,
                    float *y, int M, int N, int K, hipStream_t s)
{
    if (M % (32 * tm) != 0 || N % (32 * tn) != 0 || K < 128 || K % 128 != 0) return MI_EINVAL;   // whole tiles only
    if (tm == 8 && tn == 6) return pair::launch<8, 6, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, s);
    if (tm == 4 && tn == 8) return pair::launch<4, 8, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, s);
    return MI_EINVAL;
}


#ifdef MI_GEMM_TIMELINE
extern "C" __attribute__((visibility("default"))) int32_t mi_debug_gemm_timeline(unsigned long long *out, int32_t n)
{
    if (!out || n < 0 || n > pair::TIMELINE_WGS * 2 * 8) return MI_EINVAL;
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(pair::g_timeline), (size_t)n * 8) == hipSuccess ? MI_OK : MI_EIO;
}
#endif

template int32_t launch_pair<true>(int, int, const int8_t *, const float *, const int8_t *, const float *, int32_t *,
                                   float *, int, int, int, hipStream_t);
template int32_t launch_pair<false>(int, int, const int8_t *, const float *, const int8_t *, const float *, int32_t *,
                                    float *, int, int, int, hipStream_t);

}  // namespace mi
