// W8A8 contraction for skinny activations (decode GEMV, M <= 64):
//   acc[m,n] = sum_k qx[m,k] * qw[n,k],   y = ((float)acc * sx[m]) * sw[n]
//
// The weights [N,K] are read from HBM exactly once with 128-bit loads; the
// activation codes (at most 64 x K bytes) stay in L2.  One workgroup owns 16
// consecutive weight rows and its waves split K; a wave feeds
// v_mfma_i32_16x16x64_i8 with a 16-row x 64-byte weight fragment as the A
// operand (lane l: row l%16, bytes 16*(l/16)..+15 of the 64-byte K step) and
// the matching fragment of up to 16 tokens as the B operand.  Both operands
// use the same lane -> K mapping, and an integer dot product does not depend
// on the order of its terms, so the int32 accumulators are exact.  The waves'
// partial accumulators meet in LDS; the epilogue applies the two scales.
//
// Bound: HBM.  Algorithmic bytes per call = N*K (weights) + M*K (codes)
// + 4*M*N (output) + 4*(M+N) (scales).
#include "common.h"

namespace mi {

template <int MT, bool DEQ>
__global__ __launch_bounds__(1024) void k_w8a8_skinny(const int8_t *__restrict__ qx,
                                                      const int8_t *__restrict__ qw,
                                                      const float *__restrict__ sx,
                                                      const float *__restrict__ sw,
                                                      int32_t *__restrict__ acc_out, float *__restrict__ y,
                                                      int M, int N, int K)
{
    extern __shared__ int s_part[];  // [nwave][MT][4][64]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwave = blockDim.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int steps = K >> 6;
    const int s0 = (int)((int64_t)steps * wave / nwave), s1 = (int)((int64_t)steps * (wave + 1) / nwave);

    const int8_t *wp = qw + (int64_t)(n0 + r) * K + g * 16;
    const int8_t *xp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        int m = mt * 16 + r;
        if (m > M - 1) m = M - 1;  // rows past M are computed from a valid row and never stored
        xp[mt] = qx + (int64_t)m * K + g * 16;
    }
    v4i acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = (v4i){0, 0, 0, 0};

    constexpr int U = 4;
    int s = s0;
    for (; s + U <= s1; s += U) {
        v4i a[U];
#pragma unroll
        for (int u = 0; u < U; ++u) a[u] = *reinterpret_cast<const v4i *>(wp + (int64_t)(s + u) * 64);
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const v4i b = *reinterpret_cast<const v4i *>(xp[mt] + (int64_t)(s + u) * 64);
                acc[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[u], b, acc[mt], 0, 0, 0);
            }
        }
    }
    for (; s < s1; ++s) {
        const v4i a = *reinterpret_cast<const v4i *>(wp + (int64_t)s * 64);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const v4i b = *reinterpret_cast<const v4i *>(xp[mt] + (int64_t)s * 64);
            acc[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[mt], 0, 0, 0);
        }
    }

    // accumulator layout: lane l, register e  <->  weight row 4*(l/16)+e, token l%16
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int e = 0; e < 4; ++e) s_part[((wave * MT + mt) * 4 + e) * 64 + lane] = acc[mt][e];
    __syncthreads();

    for (int o = tid; o < 256 * MT; o += blockDim.x) {
        const int nl = o & 15, m = o >> 4;
        if (m >= M) continue;
        const int mt = m >> 4, src_lane = (nl >> 2) * 16 + (m & 15), e = nl & 3;
        int sum = 0;
        for (int w = 0; w < nwave; ++w) sum += s_part[((w * MT + mt) * 4 + e) * 64 + src_lane];
        const int n = n0 + nl;
        if constexpr (DEQ) y[(int64_t)m * N + n] = ((float)sum * sx[m]) * sw[n];
        else acc_out[(int64_t)m * N + n] = sum;
    }
}

template <bool DEQ>
int32_t launch_skinny(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc,
                      float *y, int64_t M, int64_t N, int64_t K, hipStream_t s)
{
    const int64_t groups = N / 16;
    const int cus = compute_units();
    // enough waves per compute unit to keep tens of KB of weight loads in flight
    int nwave = groups <= 2 * (int64_t)cus ? 16 : 8;
    const int64_t steps = K / 64;
    while (nwave > 1 && nwave > steps) nwave >>= 1;
    const int MT = (int)((M + 15) / 16);
    if (MT > 2 && nwave > 8) nwave = 8;  // keeps the partial sums within 32 KB of LDS
    const size_t lds = (size_t)nwave * MT * 4 * 64 * sizeof(int);
    const dim3 grid((unsigned)groups), blk((unsigned)(64 * nwave));
#define MI_SKINNY(MTT)                                                                                     \
    hipLaunchKernelGGL((k_w8a8_skinny<MTT, DEQ>), grid, blk, lds, s, qx, qw, sx, sw, acc, y, (int)M, (int)N, (int)K)
    switch (MT) {
    case 1: MI_SKINNY(1); break;
    case 2: MI_SKINNY(2); break;
    case 3: MI_SKINNY(3); break;
    case 4: MI_SKINNY(4); break;
    default: return MI_ERANGE;
    }
#undef MI_SKINNY
    return launch_status();
}

template int32_t launch_skinny<true>(const int8_t *, const float *, const int8_t *, const float *, int32_t *,
                                     float *, int64_t, int64_t, int64_t, hipStream_t);
template int32_t launch_skinny<false>(const int8_t *, const float *, const int8_t *, const float *, int32_t *,
                                      float *, int64_t, int64_t, int64_t, hipStream_t);

}  // namespace mi
