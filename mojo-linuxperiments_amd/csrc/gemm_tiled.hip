// W8A8 contraction for prefill (M > 64): LDS-tiled v_mfma_i32_16x16x64_i8.
//   acc[m,n] = sum_k qx[m,k] * qw[n,k],   y = ((float)acc * sx[m]) * sw[n]
//
// Tiling.  A workgroup of four waves (2 x 2) owns a (32*TM) x (32*TN) output
// tile; each wave owns (16*TM) x (16*TN) of it as TM*TN MFMA accumulators
// (256 registers at TM = TN = 8, which is why a SIMD holds one wave).  K is
// walked in stages of 128 bytes, double buffered in LDS.
//
// LDS layout = MFMA operand order.  A "fragment" is 16 rows x 64 K-bytes,
// stored as 1024 contiguous bytes in which lane l's 16 bytes sit at offset
// 16*l (row l%16, K-bytes 16*(l/16)..+15).  A fragment is filled by ONE
// direct-to-LDS load per wave (global_load_lds_dwordx4: every lane supplies
// its global address, the hardware writes lane l's 16 bytes at LDS base +
// 16*l) and consumed by ONE ds_read_b128 per lane with no bank conflict, no
// staging registers and no ds_write.  Both halves of a 128-byte line are
// fetched in the same stage, so every L2 line is requested once per tile.
//
// Operand roles: the weight fragment is MFMA operand A and the activation
// fragment operand B, so a lane ends up with four consecutive output channels
// of one token (registers e = 0..3 -> n = 16*tile + 4*(l/16) + e, token
// l%16) and the epilogue stores float4.
//
// Workgroup -> tile mapping is XCD-aware: hardware deals workgroup ids round
// robin over the 8 XCDs, each with a private L2, so the tile grid is cut into
// 8 rectangular parts (pm x pn) and XCD x only ever touches the rows and
// columns of part x.
//
// Bound: int8 MFMA (2*M*N*K ops).  Exact integer arithmetic.
#include "common.h"

namespace mi {

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

struct GemmGrid {
    int tiles_m, tiles_n;
    int pm, pn;  // XCD partition; pm == 0 -> plain row-major tile order
};

template <int TM, int TN, bool DEQ>
__global__ __launch_bounds__(256) void k_w8a8_tiled(const int8_t *__restrict__ qx, const int8_t *__restrict__ qw,
                                                    const float *__restrict__ sx, const float *__restrict__ sw,
                                                    int32_t *__restrict__ acc_out, float *__restrict__ y, int M,
                                                    int N, int K, GemmGrid gg)
{
    constexpr int BM = 32 * TM, BN = 32 * TN;
    constexpr int NFX = BM / 16 * 2;  // activation fragments per stage
    constexpr int NFW = BN / 16 * 2;  // weight fragments per stage
    constexpr int STAGE = (NFX + NFW) * 1024;
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, g = lane >> 4;

    int tile_m, tile_n;
    {
        const int w = blockIdx.x;
        if (gg.pm) {
            const int x = w & 7, li = w >> 3;
            const int sub_m = gg.tiles_m / gg.pm, sub_n = gg.tiles_n / gg.pn;
            (void)sub_m;
            tile_m = (x / gg.pn) * sub_m + li / sub_n;
            tile_n = (x % gg.pn) * sub_n + li % sub_n;
        } else {
            tile_m = w / gg.tiles_n;
            tile_n = w % gg.tiles_n;
        }
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    // this wave fills fragments f = wave, wave+4, ...: row tile f/2, K half f%2
    constexpr int LX = NFX / 4, LW = NFW / 4;
    const int8_t *xsrc[LX];
    const int8_t *wsrc[LW];
#pragma unroll
    for (int i = 0; i < LX; ++i) {
        const int f = wave + 4 * i;
        int row = m0 + (f >> 1) * 16 + r;
        if (row > M - 1) row = M - 1;
        xsrc[i] = qx + (int64_t)row * K + (f & 1) * 64 + g * 16;
    }
#pragma unroll
    for (int i = 0; i < LW; ++i) {
        const int f = wave + 4 * i;
        int row = n0 + (f >> 1) * 16 + r;
        if (row > N - 1) row = N - 1;
        wsrc[i] = qw + (int64_t)row * K + (f & 1) * 64 + g * 16;
    }

    auto issue = [&](int stage, int kt) {
        char *sb = smem + stage * STAGE;
        const int64_t koff = (int64_t)kt * 128;
#pragma unroll
        for (int i = 0; i < LX; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)(xsrc[i] + koff), (lptr_t)(sb + (wave + 4 * i) * 1024), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < LW; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)(wsrc[i] + koff), (lptr_t)(sb + (NFX + wave + 4 * i) * 1024), 16, 0, 0);
    };

    v4i acc[TN][TM];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int i = 0; i < TM; ++i) acc[j][i] = (v4i){0, 0, 0, 0};

    const int wm = wave >> 1, wn = wave & 1;
    const int nk = K >> 7;
    issue(0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) issue(cur ^ 1, kt + 1);
        const char *sb = smem + cur * STAGE;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            v4i xb[TM];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                xb[i] = *reinterpret_cast<const v4i *>(sb + (((wm * TM + i) * 2 + kk) * 1024) + lane * 16);
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const v4i wa = *reinterpret_cast<const v4i *>(sb + ((NFX + (wn * TN + j) * 2 + kk) * 1024) + lane * 16);
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    acc[j][i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wa, xb[i], acc[j][i], 0, 0, 0);
            }
        }
        // the next stage has landed in LDS (this wave's share: vmcnt 0; the other
        // waves' shares: barrier) and every wave is done reading this stage
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    // epilogue: lane holds n = nb + 4*g + e (e = 0..3) for token mb + r
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + (wm * TM + i) * 16 + r;
        if (m >= M) continue;
        float sxm = 0.0f;
        if constexpr (DEQ) sxm = sx[m];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + (wn * TN + j) * 16 + 4 * g;
            if (n >= N) continue;
            if constexpr (DEQ) {
                const float4 s4 = *reinterpret_cast<const float4 *>(sw + n);
                float4 o;
                o.x = ((float)acc[j][i][0] * sxm) * s4.x;
                o.y = ((float)acc[j][i][1] * sxm) * s4.y;
                o.z = ((float)acc[j][i][2] * sxm) * s4.z;
                o.w = ((float)acc[j][i][3] * sxm) * s4.w;
                *reinterpret_cast<float4 *>(y + (int64_t)m * N + n) = o;
            } else {
                *reinterpret_cast<v4i *>(acc_out + (int64_t)m * N + n) = acc[j][i];
            }
        }
    }
}

struct TileShape {
    int tm, tn;
};

template <int TM, int TN, bool DEQ>
static int32_t launch_shape(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc,
                            float *y, int M, int N, int K, hipStream_t s)
{
    constexpr int BM = 32 * TM, BN = 32 * TN;
    constexpr int LDS = 2 * (BM / 16 * 2 + BN / 16 * 2) * 1024;
    static bool attr_set = false;  // idempotent; a race only repeats the call
    if (!attr_set) {
        MI_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_w8a8_tiled<TM, TN, DEQ>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        attr_set = true;
    }
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

template <bool DEQ>
int32_t launch_tiled(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc, float *y,
                     int64_t M64, int64_t N64, int64_t K64, hipStream_t s)
{
    const int M = (int)M64, N = (int)N64, K = (int)K64;
    const int cus = compute_units();
    // pick the tile whose (rounds of tiles over the CUs) x (tile area) is least
    const TileShape shapes[] = {{8, 8}, {8, 7}, {8, 6}, {4, 8}, {4, 4}};
    int pick = 0;
    double best = 0;
    for (int i = 0; i < 5; ++i) {
        const int bm = 32 * shapes[i].tm, bn = 32 * shapes[i].tn;
        const int64_t tiles = (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
        const int per_cu = (shapes[i].tm * shapes[i].tn <= 16) ? 2 : 1;  // small tiles fit twice in LDS
        const int64_t rounds = (tiles + (int64_t)cus * per_cu - 1) / ((int64_t)cus * per_cu);
        // smaller tiles re-read more operand bytes per MFMA: mild penalty
        const double eff = (shapes[i].tm * shapes[i].tn >= 48) ? 1.0 : (shapes[i].tm * shapes[i].tn >= 32 ? 1.08 : 1.3);
        const double cost = (double)rounds * bm * bn * eff / per_cu;
        if (i == 0 || cost < best) { best = cost; pick = i; }
    }
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
