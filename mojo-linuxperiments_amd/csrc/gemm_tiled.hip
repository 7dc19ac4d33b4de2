// W8A8 contraction for prefill (M > 64): LDS-tiled v_mfma_i32_16x16x64_i8.
//   acc[m,n] = sum_k qx[m,k] * qw[n,k],   y = ((float)acc * sx[m]) * sw[n]
//
// Tiling.  A workgroup of four waves (2 x 2) owns a (32*TM) x (32*TN) output
// tile; each wave owns (16*TM) x (16*TN) of it as TM*TN MFMA accumulators held
// in AccVGPRs (192 registers at 8 x 6, so a SIMD holds one wave).  K is walked
// in stages of 128 bytes, double buffered in LDS.
//
// Global -> LDS.  Every transfer is a direct-to-LDS load
// (global_load_lds_dwordx4): one wave instruction moves 8 rows x 128 bytes,
// lane l = 8*rho + c fetching the 16-byte chunk kappa = c ^ sigma of row rho,
// and the hardware writes lane l's bytes at LDS base + 16*l.  Eight lanes per
// row means each quarter wave touches two whole 128-byte lines: measured
// 13-28 TB/s aggregate against 7-8 TB/s for the 16-rows-x-64-bytes shape that
// an MFMA fragment would suggest.  No staging registers, no ds_write.
//
// LDS -> MFMA.  A fragment (16 rows x 64 K-bytes; lane l wants row l%16, chunk
// 4*kk + l/16) is read with one ds_read_b128 per lane from two of those 1 KB
// blocks.  Measured with the bank-conflict counters: this LDS serves a
// ds_read_b128 in 4 cycles (256 B per clock) when, in each cycle, lanes 0-7 of
// one 16-lane group and lanes 8-15 of its neighbour group hit 16 distinct
// 16-byte bank groups (address mod 256), and in 8 cycles otherwise.  Rows 0-7
// of a fragment sit in the even block and rows 8-15 in the odd one, and the
// chunk position is XORed with sigma(rho, parity) = 4*parity | rho/2: rows of
// equal rho%2 (same 128-byte half of a 256-byte bank row) get four distinct
// positions inside the K half being read, and the odd block uses the other K
// half's positions, so any mix of the two blocks and of the four chunk groups
// is conflict free.
//
// Stage loop.  The MFMAs of a stage form 2*TN groups of TM instructions that
// share one weight fragment.  Fragments are fetched two groups ahead with
// explicit ds_read_b128 / s_waitcnt lgkmcnt(n) (inline asm: the compiler would
// wait for lgkmcnt(0) and expose the LDS latency in every group).  The single
// barrier of a stage sits before the last two groups: by then every wave has
// issued and drained its reads of the current buffer and its share of the next
// stage has landed (vmcnt 0), so after the barrier the next stage is visible,
// the current buffer is free, the loads of stage +2 go out at once and the
// first fragments of the next stage are fetched under the last two groups.
//
// MFMA accumulators are tied (destination == source, AccVGPR) through inline
// asm; with the builtin the register allocator rotates all accumulators
// through v_accvgpr moves in every stage.  The compiler cannot see inside the
// asm, so the one software-managed hazard that remains (VALU read of a fresh
// MFMA result) is covered by explicit wait states before the epilogue.
//
// Operand roles: the weight fragment is MFMA operand A and the activation
// fragment operand B, so a lane holds four consecutive output channels of one
// token.  The epilogue pairs neighbouring channel tiles and swaps halves
// between lanes r and r ^ 8 (DPP row_ror:8) so that one store instruction
// writes 8 rows x 128 contiguous bytes.
//
// Workgroup -> tile mapping is XCD-aware: hardware deals workgroup ids round
// robin over the 8 XCDs (measured), each with a private L2, so the tile grid
// is cut into 8 rectangular parts (pm x pn) and XCD x only ever touches the
// rows and columns of part x.
//
// Bound: int8 MFMA (2*M*N*K ops).  Exact integer arithmetic.
#include <utility>

#include "common.h"

namespace mi {

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

__device__ __forceinline__ void mfma_i8(v4i &acc, const v4i &a, const v4i &b)
{
    asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
template <int N>
__device__ __forceinline__ void wait_lgkm()
{
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory");
}
template <int OFF>
__device__ __forceinline__ void ds_read128(v4i &dst, unsigned addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
// direct-to-LDS load of 16 bytes per lane: global address = sbase + voff, LDS address = ldsaddr + 16 * lane
__device__ __forceinline__ void dma16(const int8_t *sbase, unsigned voff, unsigned ldsaddr)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(sbase), "s"(ldsaddr)
                 : "memory", "m0");
}
// how many second-half activation fragments are fetched during group g of the first half
template <int TM, int TN>
constexpr int xb1_count(int g)
{
    int c = 0;
    for (int i = 0; i < TM; ++i)
        if (i * TN / TM == g) ++c;
    return c;
}
__device__ __forceinline__ int ror8(int v) { return __builtin_amdgcn_update_dpp(v, v, 0x128, 0xf, 0xf, false); }

struct GemmGrid {
    int tiles_m, tiles_n;
    int pm, pn;  // XCD partition; pm == 0 -> plain row-major tile order
};

template <bool DEQ>
__device__ __forceinline__ void store4(float *y, int32_t *acc_out, int64_t idx, const v4i &v, float sxm, const float4 &s4)
{
    if constexpr (DEQ) {
        float4 o;
        o.x = ((float)v[0] * sxm) * s4.x;
        o.y = ((float)v[1] * sxm) * s4.y;
        o.z = ((float)v[2] * sxm) * s4.z;
        o.w = ((float)v[3] * sxm) * s4.w;
        *reinterpret_cast<float4 *>(y + idx) = o;
    } else {
        *reinterpret_cast<v4i *>(acc_out + idx) = v;
    }
}

// LDS budget: two activation buffers and, where 160 KB allow it, three weight buffers (a small tile keeps
// two so that two workgroups share a compute unit)
template <int TM, int TN>
struct TiledCfg {
    static constexpr int NBX = 4 * TM, NBW = 4 * TN;
    static constexpr int NWB = (TM * TN <= 16) ? 2 : ((2 * NBX + 3 * NBW <= 160) ? 3 : 2);
    static constexpr int LDS = (2 * NBX + NWB * NBW) * 1024;
};

template <int TM, int TN, bool DEQ>
__global__ __launch_bounds__(256) void k_w8a8_tiled(const int8_t *__restrict__ qx, const int8_t *__restrict__ qw,
                                                    const float *__restrict__ sx, const float *__restrict__ sw,
                                                    int32_t *__restrict__ acc_out, float *__restrict__ y, int M,
                                                    int N, int K, GemmGrid gg)
{
    constexpr int BM = 32 * TM, BN = 32 * TN;
    constexpr int NBX = BM / 8, NBW = BN / 8;  // 1 KB blocks (8 rows x 128 B) per stage
    constexpr int G = 2 * TN;                  // MFMA groups per stage
    constexpr int NWB = TiledCfg<TM, TN>::NWB;
    constexpr int XSTAGE = NBX * 1024, WSTAGE = NBW * 1024, XAREA = 2 * XSTAGE;
    constexpr int R = (G % 3 == 0) ? 3 : ((G % 4 == 0) ? 4 : 3);  // weight fragment registers in rotation
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

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

    // load side: this wave fills blocks b = wave, wave+4, ... of each stage.  Addresses are a uniform
    // 64-bit base (SGPR pair, advanced per stage) plus a 32-bit per-lane offset: the scalar-base form
    // occupies the wave's issue slot for fewer cycles than a 64-bit VGPR address, and with one wave
    // per SIMD every cycle a load holds the issue slot is a cycle the MFMA pipe is not fed.
    constexpr int LX = NBX / 4, LW = NBW / 4;
    unsigned vx[LX], vw[LW];
    {
        const int rho = lane >> 3, c = lane & 7;
#pragma unroll
        for (int i = 0; i < LX; ++i) {
            const int b = wave + 4 * i;
            const int sigma = ((b & 1) << 2) | (rho >> 1);
            int row = b * 8 + rho;
            if (row > M - 1 - m0) row = M - 1 - m0;  // rows past the edge are computed from a valid row and never stored
            vx[i] = (unsigned)row * (unsigned)K + (unsigned)((c ^ sigma) << 4);
        }
#pragma unroll
        for (int i = 0; i < LW; ++i) {
            const int b = wave + 4 * i;
            const int sigma = ((b & 1) << 2) | (rho >> 1);
            int row = b * 8 + rho;
            if (row > N - 1 - n0) row = N - 1 - n0;
            vw[i] = (unsigned)row * (unsigned)K + (unsigned)((c ^ sigma) << 4);
        }
    }
    const int8_t *const xtile = qx + (int64_t)m0 * K;
    const int8_t *const wtile = qw + (int64_t)n0 * K;
    const unsigned lds_base = (unsigned)(uintptr_t)(lptr_t)smem;
    const unsigned lds_x = lds_base + wave * 1024, lds_w = lds_base + XAREA + wave * 1024;
    // the activation loads of a stage are scheduled over SPX groups, the weight loads over SPW groups
    constexpr int SPX = (TN - 2 < LX) ? TN - 2 : LX, SPW = LW;
    auto issue_x = [&](auto P, unsigned buf, int kt) {
        const int8_t *src = xtile + (int64_t)kt * 128;
        static_for<LX>([&](auto I) {
            constexpr int i = decltype(I)::value;
            if constexpr (decltype(P)::value < 0 || i * SPX / LX == decltype(P)::value) dma16(src, vx[i], lds_x + buf + i * 4096);
        });
    };
    auto issue_w = [&](auto P, unsigned buf, int kt) {
        const int8_t *src = wtile + (int64_t)kt * 128;
        static_for<LW>([&](auto I) {
            constexpr int i = decltype(I)::value;
            if constexpr (decltype(P)::value < 0 || i * SPW / LW == decltype(P)::value) dma16(src, vw[i], lds_w + buf + i * 4096);
        });
    };
    constexpr std::integral_constant<int, -1> ALL{};

    // read side
    const int r = lane & 15, g_ = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;
    unsigned roff0, roff1;
    {
        const int rho = r & 7, bpar = r >> 3;
        const int sigma = (bpar << 2) | (rho >> 1);
        roff0 = bpar * 1024 + ((8 * rho + ((0 + g_) ^ sigma)) << 4);
        roff1 = bpar * 1024 + ((8 * rho + ((4 + g_) ^ sigma)) << 4);
    }
    const unsigned xo = lds_base + wm * TM * 2048, wo = lds_base + XAREA + wn * TN * 2048;

    v4i acc[TN][TM];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int i = 0; i < TM; ++i) acc[j][i] = (v4i){0, 0, 0, 0};
    v4i xb0[TM], xb1[TM], wa[R];

    // The scales of the epilogue are requested before the first stage: a load issued between the stores would wait
    // for every store before it (the memory counter is shared and counts in order), and one issued after the loop
    // would put a memory round trip between the last MFMA and the first store.  28 registers for the whole loop.
    const bool lo = r < 8;
    float sxA[TM], sxB[TM], sxO[TM];
    float4 swP[(TN + 1) / 2];
    if constexpr (DEQ) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int mrow = m0 + (wm * TM + i) * 16;
            const int mA = mrow + (r & 7), mB = mrow + 8 + (r & 7), mO = mrow + r;
            sxA[i] = sx[mA < M ? mA : M - 1];
            sxB[i] = sx[mB < M ? mB : M - 1];
            if constexpr (TN & 1) sxO[i] = sx[mO < M ? mO : M - 1];
        }
#pragma unroll
        for (int j = 0; j < TN; j += 2) {
            int n = n0 + (wn * TN + j) * 16 + ((!lo && j + 1 < TN) ? 16 : 0) + 4 * g_;
            if (n > N - 4) n = N - 4;
            swP[j / 2] = *reinterpret_cast<const float4 *>(sw + n);
        }
    }

    const int nk = K >> 7;
    // stage s lives in activation buffer s % 2 and weight buffer s % NWB; the offsets rotate with the stage
    unsigned xcur = 0, xnxt = XSTAGE;
    unsigned wcur = 0, wnxt = WSTAGE, wnn = (NWB == 3) ? 2 * WSTAGE : 0;
    issue_x(ALL, 0u, 0);
    issue_w(ALL, 0u, 0);
    if (nk > 1) {
        issue_w(ALL, wnxt, 1);
        issue_x(ALL, xnxt, 1);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LX + LW) : "memory");
    } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
    if constexpr (NWB == 3) {
        if (nk > 2) {
            issue_w(std::integral_constant<int, 0>{}, wnn, 2);
            if constexpr (SPW > 1) issue_w(std::integral_constant<int, 1>{}, wnn, 2);
        }
    }
    {   // first fragments of stage 0
        const unsigned ax0 = xo + roff0, aw0 = wo + roff0;
        static_for<TM>([&](auto I) { ds_read128<decltype(I)::value * 2048>(xb0[decltype(I)::value], ax0); });
        ds_read128<0>(wa[0], aw0);
        ds_read128<2048>(wa[1], aw0);
    }
    for (int kt = 0; kt < nk; ++kt) {
        const unsigned ax1 = xo + xcur + roff1, aw0 = wo + wcur + roff0, aw1 = wo + wcur + roff1;
        const unsigned nax0 = xo + xnxt + roff0, naw0 = wo + wnxt + roff0;
        const bool more = kt + 2 < nk;
        static_for<G>([&](auto GG) {
            constexpr int g = decltype(GG)::value;
            constexpr int kk = g / TN, j = g % TN;
            // weight loads continue from the two slots used under the previous stage's last two groups
            if constexpr (g + 2 < SPW) {
                if constexpr (NWB == 3) {
                    if (more) issue_w(std::integral_constant<int, g + 2>{}, wnn, kt + 2);
                } else {
                    if (kt > 0 && kt + 1 < nk) issue_w(std::integral_constant<int, g + 2>{}, wnxt, kt + 1);
                }
            }
            if constexpr (g > TN && g - TN < SPX && g < G - 2) {
                if (more) issue_x(std::integral_constant<int, g - TN>{}, xcur, kt + 2);
            }
            if constexpr (g == G - 2) {
                // all reads of the current buffers have been issued: drain them and this wave's share of
                // the next stage (loads return in order, so the loads of later stages may stay in flight)
                if (more) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(LX + (NWB == 3 ? LW : 0)) : "memory");
                else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                __syncthreads();
                if (kt + NWB < nk) issue_w(std::integral_constant<int, 0>{}, wcur, kt + NWB);
                static_for<TM>([&](auto I) { ds_read128<decltype(I)::value * 2048>(xb0[decltype(I)::value], nax0); });
                ds_read128<0>(wa[G % R], naw0);
            } else if constexpr (g == G - 1) {
                if constexpr (SPW > 1) {
                    if (kt + NWB < nk) issue_w(std::integral_constant<int, 1>{}, wcur, kt + NWB);
                }
                ds_read128<2048>(wa[(G + 1) % R], naw0);
            } else {
                if constexpr (kk == 0) {
                    static_for<TM>([&](auto I) {
                        constexpr int i = decltype(I)::value;
                        if constexpr (i * TN / TM == j) ds_read128<i * 2048>(xb1[i], ax1);
                    });
                }
                constexpr int g2 = g + 2;  // <= G - 1
                ds_read128<(g2 % TN) * 2048>(wa[g2 % R], (g2 / TN) ? aw1 : aw0);
                // LDS returns in order: allow the reads issued after wa[g % R] to stay in flight
                constexpr int c_prev = (kk == 0 && g >= 1) ? xb1_count<TM, TN>(g - 1) : 0;
                constexpr int c_cur = (kk == 0) ? xb1_count<TM, TN>(g) : 0;
                wait_lgkm<2 + c_prev + c_cur>();
                if constexpr (g == TN) {
                    // this wave now holds all its activation fragments of the stage in registers; once
                    // every wave does, the activation buffer is free for the stage after next
                    __builtin_amdgcn_s_barrier();
                    if (more) issue_x(std::integral_constant<int, 0>{}, xcur, kt + 2);
                }
            }
#pragma unroll
            for (int i = 0; i < TM; ++i) mfma_i8(acc[j][i], wa[g % R], kk ? xb1[i] : xb0[i]);
        });
        // the next stage numbers its groups from 0 again
        if constexpr (G % R != 0) {
            wait_lgkm<0>();
            const v4i t0 = wa[G % R], t1 = wa[(G + 1) % R];
            wa[0] = t0;
            wa[1] = t1;
        }
        {
            const unsigned t = xcur; xcur = xnxt; xnxt = t;
            if constexpr (NWB == 3) { const unsigned u = wcur; wcur = wnxt; wnxt = wnn; wnn = u; }
            else { const unsigned u = wcur; wcur = wnxt; wnxt = u; }
        }
    }
    // drain the trailing fragment reads; 2 x 16 wait states cover the longest MFMA-result -> VALU-read hazard
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\ns_nop 15\ns_nop 15" ::: "memory");

    // epilogue: lane holds channels nb + 4*g_ .. +3 of token mrow + r for each (i, j); interior tiles take a
    // branch-free path: with divergent branches between the stores the compiler
    // can no longer count how many are in flight and falls back to waiting for each one
    auto emit = [&](auto CHECKED) {
        constexpr bool checked = decltype(CHECKED)::value;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int mrow = m0 + (wm * TM + i) * 16;
            const int mA = mrow + (r & 7), mB = mrow + 8 + (r & 7);
#pragma unroll
            for (int j = 0; j + 1 < TN; j += 2) {
                const int nb0 = n0 + (wn * TN + j) * 16;
                const v4i a0 = acc[j][i], a1 = acc[j + 1][i];
                v4i t0, t1;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    t0[e] = ror8(a0[e]);
                    t1[e] = ror8(a1[e]);
                }
                const v4i vA = lo ? a0 : t1;  // rows 0-7:  lanes r<8 tile j (own), lanes r>=8 tile j+1 (from lane r-8)
                const v4i vB = lo ? t0 : a1;  // rows 8-15: lanes r>=8 tile j+1 (own), lanes r<8 tile j (from lane r+8)
                const int n = nb0 + (lo ? 0 : 16) + 4 * g_;
                if (!checked || n < N) {
                    if (!checked || mA < M) store4<DEQ>(y, acc_out, (int64_t)mA * N + n, vA, sxA[i], swP[j / 2]);
                    if (!checked || mB < M) store4<DEQ>(y, acc_out, (int64_t)mB * N + n, vB, sxB[i], swP[j / 2]);
                }
            }
            if constexpr (TN & 1) {
                constexpr int j = TN - 1;
                const int m = mrow + r;
                const int n = n0 + (wn * TN + j) * 16 + 4 * g_;
                if (!checked || (m < M && n < N)) store4<DEQ>(y, acc_out, (int64_t)m * N + n, acc[j][i], sxO[i], swP[j / 2]);
            }
        }
    };
    if (m0 + BM <= M && n0 + BN <= N) emit(std::false_type{});
    else emit(std::true_type{});
}

struct TileShape {
    int tm, tn;
};

template <int TM, int TN, bool DEQ>
static int32_t launch_shape(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc,
                            float *y, int M, int N, int K, hipStream_t s)
{
    constexpr int BM = 32 * TM, BN = 32 * TN;
    constexpr int LDS = TiledCfg<TM, TN>::LDS;
    // ragged M and N are the kernel's to clamp; the K loop moves whole 128-byte stages and the stores whole
    // 16-column groups, which nothing behind this line checks again
    if (M <= 0 || N <= 0 || N % 16 != 0 || K < 128 || K % 128 != 0) return MI_EINVAL;
    MI_LDS_OPT_IN((&k_w8a8_tiled<TM, TN, DEQ>), LDS);
    GemmGrid gg;
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
    const dim3 grid((unsigned)(gg.tiles_m * gg.tiles_n)), blk(256);
    hipLaunchKernelGGL((k_w8a8_tiled<TM, TN, DEQ>), grid, blk, LDS, s, qx, qw, sx, sw, acc, y, M, N, K, gg);
    return launch_status();
}

// gemm_pair.hip
template <bool DEQ>
int32_t launch_pair(int tm, int tn, const int8_t *, const float *, const int8_t *, const float *, int32_t *, float *, int,
                    int, int, hipStream_t);

template <bool DEQ>
int32_t launch_tiled(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc, float *y,
                     int64_t M64, int64_t N64, int64_t K64, hipStream_t s)
{
    const int M = (int)M64, N = (int)N64, K = (int)K64;
    const int cus = compute_units();
    // pick the tile with the least (rounds of tiles over the chip) x (work a compute unit does per round)
    const TileShape shapes[] = {{8, 8}, {8, 7}, {8, 6}, {4, 8}, {4, 4}};
    int pick = 0;
    double best = 0;
    for (int i = 0; i < 5; ++i) {
        const int bm = 32 * shapes[i].tm, bn = 32 * shapes[i].tn;
        const int64_t tiles = (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
        const int per_cu = (shapes[i].tm * shapes[i].tn <= 16) ? 2 : 1;  // small tiles fit twice in LDS
        const int64_t slots = (int64_t)cus * per_cu;
        const int64_t rounds = (tiles + slots - 1) / slots;
        // co-resident tiles share the compute unit's MFMA and LDS; smaller wave tiles read more LDS bytes per MFMA
        const int area = shapes[i].tm * shapes[i].tn;
        const double eff = area >= 48 ? 1.0 : (area >= 32 ? 1.08 : 1.5);
        const double cost = (double)rounds * per_cu * bm * bn * eff;
        if (i == 0 || cost < best) { best = cost; pick = i; }
    }
    // one tile per compute unit of a shape that divides evenly: two waves per SIMD on the same wave tile
    if ((pick == 2 || pick == 3) && M % (32 * shapes[pick].tm) == 0 && N % (32 * shapes[pick].tn) == 0)
        return launch_pair<DEQ>(shapes[pick].tm, shapes[pick].tn, qx, sx, qw, sw, acc, y, M, N, K, s);
    switch (pick) {
    case 0: return launch_shape<8, 8, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, s);
    case 1: return launch_shape<8, 7, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, s);
    case 2: return launch_shape<8, 6, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, s);
    case 3: return launch_shape<4, 8, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, s);
    default: return launch_shape<4, 4, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, s);
    }
}

template int32_t launch_tiled<true>(const int8_t *, const float *, const int8_t *, const float *, int32_t *, float *,
                                    int64_t, int64_t, int64_t, hipStream_t);
template int32_t launch_tiled<false>(const int8_t *, const float *, const int8_t *, const float *, int32_t *, float *,
                                     int64_t, int64_t, int64_t, hipStream_t);

}  // namespace mi
