// MoE layer (workload elements a9 router, a10 dispatch, a11 grouped expert FFN).
//
//   route    : logits = x . wr^T (fixed fp32 order), top-k on logits, softmax over picks
//   dispatch : stable grouping of the T*topk (token, slot) pairs by expert
//   ffn      : qx = quant(FWHT128(x))                       once per token
//              per expert segment: g,u = qx . wg^T, qx . wu^T   (int8 MFMA, exact)
//                                  h = silu(g) * u              (fp32)  -> sorted order
//              hq = quant(FWHT256(h))                           per pair
//              per expert segment: out[pair] = hq . wd^T        (int8 MFMA, exact)
//              y[token] = sum_slot w[token,slot] * out[pair]    (fixed order, no atomics)
//
// The expert GEMMs are weight-streaming bound (each expert sees ~32 rows): a
// workgroup owns 16 gate + 16 up rows (or 32 down rows) of one expert, streams
// them from HBM once through wave-private LDS rings, and walks the expert's
// tokens 32 at a time with the gathered activation codes as MFMA B fragments.
// Waves split K; partial accumulators meet in LDS.
//
// Bound: HBM on the int8 expert weights, E * 3 * H * I bytes per layer call.
#include "common.h"
#include "fwht_core.h"

namespace mi {
namespace moe {

constexpr int MAX_TOPK = 8;
static int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }
constexpr int64_t DISPATCH_MAX_WORDS = 36864;  // 144 KB of the 160 KB LDS

__device__ __forceinline__ float shfl_xor_f(float v, int m) { return __shfl_xor(v, m, 64); }

// ---------------------------------------------------------------- a9 router
// Workgroup = E/16 waves, 4 tokens.  Wave eg owns experts 16*eg .. 16*eg+15 for
// the 4 tokens: 64 (token, expert) dot products.  Lane l accumulates, for every
// one of them, the terms k = 256*j + 4*l + c (j ascending, c = 0..3) with one
// FMA each; the 64 lanes' partial sums are then combined by the butterfly
// l ^ 32, 16, 8, 4, 2, 1.  Instead of six shuffles per dot product, the
// butterfly is run "transposed": in the round with offset `off` a lane hands
// the half of its dot products whose index bit differs from its own lane bit
// to its partner and keeps the other half, so each addition joins exactly the
// two operands the plain butterfly would join (float add is commutative) and
// 63 shuffles finish 64 dot products.  Lane l ends with pair l.
template <int OFF, int N, int NP>
__device__ __forceinline__ void fold(float (&p)[NP], int lane)
{
    const bool hi = (lane & OFF) != 0;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const float keep = hi ? p[i + N] : p[i];
        const float send = hi ? p[i] : p[i + N];
        p[i] = keep + shfl_xor_f(send, OFF);
    }
}

// grid = (T/16, E/EW): a workgroup of 4 waves covers 16 tokens x EW experts, so the router weights are read
// T/16 times and the activations E/EW times in all (both from L2), and every compute unit gets work.
// CQ > 0: the kernel also rotates (block 128) and quantizes the token rows for the expert FFN, a wave per row with CQ
// chunks per lane (H = 512 * CQ at most), the arithmetic of the stand-alone quantizer: the 16 tokens of a group are
// dealt to the waves of the group's workgroups, so that the layer launches one kernel less.
// EW = 8: a wave owns 8 experts for its 4 tokens (32 dot products a lane, half the registers, twice the workgroups):
// two waves share a SIMD where EW = 16 leaves one alone with its memory round trips (cfg4: 17.2 -> 13.8 us; four
// experts a wave, or loads two rounds ahead in three register sets, measured the same 13.8).  The first butterfly
// round (offset 32) is then the plain one; lanes l and l ^ 32 end with the same pair.
template <int CQ, int EW>
__global__ __launch_bounds__(256) void k_moe_logits(const float *__restrict__ x, const float *__restrict__ wr,
                                                    float *__restrict__ logits, int T, int H, int E,
                                                    int8_t *__restrict__ qx, float *__restrict__ sx)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t0 = blockIdx.x * 16 + wave * 4;
    const int e0 = blockIdx.y * EW;

    // the token row this wave quantizes (if any) is requested first: its loads then fly under the logits' rounds
    // instead of costing a memory round trip after them
    constexpr int LPB = 16;
    constexpr int CQR = CQ > 0 ? CQ : 1;
    const int jq = lane % LPB, nchunk = H / 8;
    const int qtt = (int)blockIdx.y * 4 + wave;                 // the workgroups of a token group deal its 16 rows
    const int qrow = blockIdx.x * 16 + qtt;
    const bool has_row = CQ > 0 && qtt < 16 && qrow < T;        // whole wave
    float v[CQR][8];
    int base[CQR];
    if constexpr (CQ > 0) {
        const float *xrow = x + (int64_t)min(qrow, T - 1) * H;
#pragma unroll
        for (int i = 0; i < CQ; ++i) {
            const int c = lane + i * 64;
            base[i] = (c / LPB) * 128 + 4 * jq;
            if (has_row && c < nchunk) {
                const float4 lo = *reinterpret_cast<const float4 *>(xrow + base[i]);
                const float4 hi = *reinterpret_cast<const float4 *>(xrow + base[i] + 64);
                v[i][0] = lo.x; v[i][1] = lo.y; v[i][2] = lo.z; v[i][3] = lo.w;
                v[i][4] = hi.x; v[i][5] = hi.y; v[i][6] = hi.z; v[i][7] = hi.w;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[i][e] = 0.0f;
            }
        }
    }

    float p[4 * EW];
#pragma unroll
    for (int i = 0; i < 4 * EW; ++i) p[i] = 0.0f;
    const float *xr[4];
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) xr[tt] = x + (int64_t)min(t0 + tt, T - 1) * H + 4 * lane;
    const float *wp = wr + (int64_t)e0 * H + 4 * lane;
    // Eight experts at a time: while the 128 FMAs of one half run, the weights of the next half (and, behind a
    // second half, the token rows of the next round) are already on their way; with one wave per SIMD the loop is
    // otherwise a chain of memory round trips.  Every dot product still takes its terms in the same order.
    const int nj = H / 256;
    if constexpr (EW == 16) {
        float4 xv[4], xn[4], wa[8], wb[8];
    #pragma unroll
        for (int tt = 0; tt < 4; ++tt) xv[tt] = *reinterpret_cast<const float4 *>(xr[tt]);
    #pragma unroll
        for (int e = 0; e < 8; ++e) wa[e] = *reinterpret_cast<const float4 *>(wp + (int64_t)e * H);
        for (int j = 0; j < nj; ++j) {
    #pragma unroll
            for (int e = 0; e < 8; ++e) wb[e] = *reinterpret_cast<const float4 *>(wp + (int64_t)(8 + e) * H + 256 * j);
    #pragma unroll
            for (int tt = 0; tt < 4; ++tt)
    #pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float a = p[tt * 16 + e];
                    a = __builtin_fmaf(xv[tt].x, wa[e].x, a);
                    a = __builtin_fmaf(xv[tt].y, wa[e].y, a);
                    a = __builtin_fmaf(xv[tt].z, wa[e].z, a);
                    a = __builtin_fmaf(xv[tt].w, wa[e].w, a);
                    p[tt * 16 + e] = a;
                }
            const int jn = min(j + 1, nj - 1);   // (the last round fetches itself again: no branch around loads)
    #pragma unroll
            for (int e = 0; e < 8; ++e) wa[e] = *reinterpret_cast<const float4 *>(wp + (int64_t)e * H + 256 * jn);
    #pragma unroll
            for (int tt = 0; tt < 4; ++tt) xn[tt] = *reinterpret_cast<const float4 *>(xr[tt] + 256 * jn);
    #pragma unroll
            for (int tt = 0; tt < 4; ++tt)
    #pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float a = p[tt * 16 + 8 + e];
                    a = __builtin_fmaf(xv[tt].x, wb[e].x, a);
                    a = __builtin_fmaf(xv[tt].y, wb[e].y, a);
                    a = __builtin_fmaf(xv[tt].z, wb[e].z, a);
                    a = __builtin_fmaf(xv[tt].w, wb[e].w, a);
                    p[tt * 16 + 8 + e] = a;
                }
    #pragma unroll
            for (int tt = 0; tt < 4; ++tt) xv[tt] = xn[tt];
        }
    } else {
        // one group of eight experts: the next round's weights and token rows are requested before this round's
        // 128 FMAs
        float4 xv[4], xn[4], wa[8], wn[8];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) xv[tt] = *reinterpret_cast<const float4 *>(xr[tt]);
#pragma unroll
        for (int e = 0; e < 8; ++e) wa[e] = *reinterpret_cast<const float4 *>(wp + (int64_t)e * H);
        for (int j = 0; j < nj; ++j) {
            const int jn = min(j + 1, nj - 1);   // (the last round fetches itself again: no branch around loads)
#pragma unroll
            for (int e = 0; e < 8; ++e) wn[e] = *reinterpret_cast<const float4 *>(wp + (int64_t)e * H + 256 * jn);
#pragma unroll
            for (int tt = 0; tt < 4; ++tt) xn[tt] = *reinterpret_cast<const float4 *>(xr[tt] + 256 * jn);
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float a = p[tt * 8 + e];
                    a = __builtin_fmaf(xv[tt].x, wa[e].x, a);
                    a = __builtin_fmaf(xv[tt].y, wa[e].y, a);
                    a = __builtin_fmaf(xv[tt].z, wa[e].z, a);
                    a = __builtin_fmaf(xv[tt].w, wa[e].w, a);
                    p[tt * 8 + e] = a;
                }
#pragma unroll
            for (int e = 0; e < 8; ++e) wa[e] = wn[e];
#pragma unroll
            for (int tt = 0; tt < 4; ++tt) xv[tt] = xn[tt];
        }
    }
    if constexpr (EW == 16) {
        fold<32, 32>(p, lane);
        fold<16, 16>(p, lane);
        fold<8, 8>(p, lane);
        fold<4, 4>(p, lane);
        fold<2, 2>(p, lane);
        fold<1, 1>(p, lane);
        // lane l now holds pair l: token l/16, expert e0 + l%16
        const int t = t0 + (lane >> 4);
        if (t < T) logits[(int64_t)t * E + e0 + (lane & 15)] = p[0];
    } else {
        static_assert(EW == 8, "experts per wave");
#pragma unroll
        for (int i = 0; i < 32; ++i) p[i] = p[i] + shfl_xor_f(p[i], 32);
        fold<16, 16>(p, lane);
        fold<8, 8>(p, lane);
        fold<4, 4>(p, lane);
        fold<2, 2>(p, lane);
        fold<1, 1>(p, lane);
        // lanes l and l ^ 32 now hold pair l % 32: token (l % 32) / 8, expert e0 + l % 8
        const int t = t0 + ((lane & 31) >> 3);
        if (lane < 32 && t < T) logits[(int64_t)t * E + e0 + (lane & 7)] = p[0];
    }
    if constexpr (CQ > 0) {
        if (has_row) {
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < CQ; ++i) {
                fwht_chunk<128>(v[i], jq);
                amax = fmaxf(amax, abs8(v[i]));
            }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
            const float sc = (amax == 0.0f) ? 1.0f : amax / 127.0f;
            const float inv = (amax == 0.0f) ? 0.0f : 127.0f / amax;
            if (lane == 0) sx[qrow] = sc;
            int8_t *qr = qx + (int64_t)qrow * H;
#pragma unroll
            for (int i = 0; i < CQ; ++i) {
                if (lane + i * 64 < nchunk) {
                    *reinterpret_cast<uint32_t *>(qr + base[i]) = quant4(v[i][0], v[i][1], v[i][2], v[i][3], inv);
                    *reinterpret_cast<uint32_t *>(qr + base[i] + 64) = quant4(v[i][4], v[i][5], v[i][6], v[i][7], inv);
                }
            }
        }
        // fewer than four expert groups: a wave has further rows of the token group to do
        for (int tt = qtt + (int)gridDim.y * 4; tt < 16; tt += (int)gridDim.y * 4) {
            const int row = blockIdx.x * 16 + tt;
            if (row >= T) break;   // whole wave
            const float *xrow = x + (int64_t)row * H;
#pragma unroll
            for (int i = 0; i < CQ; ++i) {
                if (lane + i * 64 < nchunk) {
                    const float4 lo = *reinterpret_cast<const float4 *>(xrow + base[i]);
                    const float4 hi = *reinterpret_cast<const float4 *>(xrow + base[i] + 64);
                    v[i][0] = lo.x; v[i][1] = lo.y; v[i][2] = lo.z; v[i][3] = lo.w;
                    v[i][4] = hi.x; v[i][5] = hi.y; v[i][6] = hi.z; v[i][7] = hi.w;
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[i][e] = 0.0f;
                }
            }
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < CQ; ++i) {
                fwht_chunk<128>(v[i], jq);
                amax = fmaxf(amax, abs8(v[i]));
            }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
            const float sc = (amax == 0.0f) ? 1.0f : amax / 127.0f;
            const float inv = (amax == 0.0f) ? 0.0f : 127.0f / amax;
            if (lane == 0) sx[row] = sc;
            int8_t *qr = qx + (int64_t)row * H;
#pragma unroll
            for (int i = 0; i < CQ; ++i) {
                if (lane + i * 64 < nchunk) {
                    *reinterpret_cast<uint32_t *>(qr + base[i]) = quant4(v[i][0], v[i][1], v[i][2], v[i][3], inv);
                    *reinterpret_cast<uint32_t *>(qr + base[i] + 64) = quant4(v[i][4], v[i][5], v[i][6], v[i][7], inv);
                }
            }
        }
    }
}

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float readlane_f(float v, int l)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}

// one wave per token: k rounds of (wave-wide max, lowest index among the lanes that hold it); lane l holds
// experts l, l+64, l+128, l+192.  Ties go to the lower expert index; picks come out by descending logit.
__global__ __launch_bounds__(256) void k_moe_topk(const float *__restrict__ logits, int32_t *__restrict__ idx,
                                                  float *__restrict__ w, int T, int E, int topk)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t = blockIdx.x * 4 + wave;
    if (t >= T) return;   // whole wave
    float mine[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int i = lane + 64 * u;
        mine[u] = i < E ? logits[(int64_t)t * E + i] : -INFINITY;
    }
    float top[MAX_TOPK];
    int pick_lane = 0;       // lane s keeps pick s
    for (int s = 0; s < topk; ++s) {
        // wave-wide maximum: four DPP steps leave every 16-lane row with its own maximum, four scalar reads join the
        // rows (a chain of cross-lane permutes costs five times as many cycles, and this loop is all latency)
        float v = fmaxf(fmaxf(mine[0], mine[1]), fmaxf(mine[2], mine[3]));
        v = fmaxf(v, dpp_f<0xB1>(v));    // quad_perm [1,0,3,2]
        v = fmaxf(v, dpp_f<0x4E>(v));    // quad_perm [2,3,0,1]
        v = fmaxf(v, dpp_f<0x124>(v));   // row_ror:4
        v = fmaxf(v, dpp_f<0x128>(v));   // row_ror:8
        v = fmaxf(fmaxf(readlane_f(v, 0), readlane_f(v, 16)), fmaxf(readlane_f(v, 32), readlane_f(v, 48)));
        // lowest expert index holding v: experts of slot u are 64u .. 64u+63, so the first non-empty ballot wins
        int win = -1;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const unsigned long long bal = __ballot(mine[u] == v);
            if (win < 0 && bal) {
                const int wl = __ffsll((long long)bal) - 1;
                win = wl + 64 * u;
                if (lane == wl) mine[u] = -INFINITY;   // taken
            }
        }
        if (lane == s) pick_lane = win;
#pragma unroll
        for (int q = 0; q < MAX_TOPK; ++q)
            if (q == s) top[q] = v;
    }
    // lane s evaluates e_s = expf(l_s - l_0) once; the sum runs over the picks in pick order, as the oracle's does
    float mine_top = top[0];
#pragma unroll
    for (int q = 1; q < MAX_TOPK; ++q)
        if (q == lane) mine_top = top[q];
    const float e = lane < topk ? expf(mine_top - top[0]) : 0.0f;
    float sum = 0.0f;
#pragma unroll
    for (int q = 0; q < MAX_TOPK; ++q)
        if (q < topk) sum = sum + readlane_f(e, q);
    if (lane < topk) {
        idx[(int64_t)t * topk + lane] = pick_lane;
        w[(int64_t)t * topk + lane] = e / sum;
    }
}

// -------------------------------------------------------------- a10 dispatch
// One workgroup.  bm[e][t/32] bit t%32 = "token t picked expert e" (a token
// picks an expert at most once), so the stable rank of pair (t, slot) inside
// its expert is the number of set bits below t in row e.
// order (optional): expert ids by descending segment size, so that the grouped GEMMs can start their longest
// workgroups first.
__global__ __launch_bounds__(1024) void k_moe_dispatch(const int32_t *__restrict__ idx, int32_t *__restrict__ perm,
                                                       int32_t *__restrict__ seg_off, int32_t *__restrict__ order,
                                                       int T, int E, int topk)
{
    extern __shared__ uint32_t s_dyn[];
    const int W = (T + 31) >> 5;
    uint32_t *bm = s_dyn;                 // [E][W]
    uint32_t *pre = s_dyn + E * W;        // [E][W] exclusive popcount prefix
    int *seg = reinterpret_cast<int *>(s_dyn + 2 * E * W);  // [E+1]
    const int tid = threadIdx.x, nt = blockDim.x;
    const int P = T * topk;
    for (int i = tid; i < E * W; i += nt) bm[i] = 0u;
    // a thread's pairs stay in registers between the two passes when they are few (one global round trip less)
    constexpr int KEEP = 8;
    const bool keep = P <= KEEP * nt;
    int mine[KEEP];
    if (keep) {
#pragma unroll
        for (int i = 0; i < KEEP; ++i) {
            const int pr = tid + i * nt;
            mine[i] = pr < P ? idx[pr] : -1;
        }
    }
    __syncthreads();
    if (keep) {
#pragma unroll
        for (int i = 0; i < KEEP; ++i) {
            const int e = mine[i], t = (tid + i * nt) / topk;
            if (e >= 0 && e < E) atomicOr(&bm[e * W + (t >> 5)], 1u << (t & 31));
        }
    } else {
        for (int pr = tid; pr < P; pr += nt) {
            const int e = idx[pr], t = pr / topk;
            if (e >= 0 && e < E) atomicOr(&bm[e * W + (t >> 5)], 1u << (t & 31));
        }
    }
    __syncthreads();
    for (int e = tid; e < E; e += nt) {
        int c = 0;
        for (int wd = 0; wd < W; ++wd) {
            pre[e * W + wd] = (uint32_t)c;
            c += __popc(bm[e * W + wd]);
        }
        seg[e + 1] = c;
    }
    __syncthreads();
    // exclusive scan of the E counts by one wave: lane l sums its run of ceil(E/64) counts, the wave scans the 64
    // run totals with shuffles, the lane writes its run back (a serial loop over E through LDS costs a dependent
    // LDS round trip per expert)
    if (tid < 64) {
        const int run = (E + 63) / 64;
        const int lo = min(tid * run, E), hi = min(lo + run, E);
        int sum = 0;
        for (int e = lo; e < hi; ++e) sum += seg[e + 1];
        int incl = sum;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int v = __shfl_up(incl, off, 64);
            if (tid >= off) incl += v;
        }
        int acc = incl - sum;
        if (tid == 0) seg[0] = 0;
        for (int e = lo; e < hi; ++e) {
            acc += seg[e + 1];
            seg[e + 1] = acc;
        }
    }
    __syncthreads();
    for (int e = tid; e <= E; e += nt) seg_off[e] = seg[e];
    if (order) {
        // rank of expert e among the counts (descending, ties by index): 8 lanes share an expert
        for (int e0 = 0; e0 < E; e0 += nt / 8) {
            const int e = e0 + (tid >> 3), part = tid & 7;
            int rank = 0;
            if (e < E) {
                const int c = seg[e + 1] - seg[e];
                for (int o = part; o < E; o += 8) {
                    const int co = seg[o + 1] - seg[o];
                    rank += (co > c || (co == c && o < e)) ? 1 : 0;
                }
            }
            rank += __shfl_xor(rank, 1, 64);
            rank += __shfl_xor(rank, 2, 64);
            rank += __shfl_xor(rank, 4, 64);
            if (e < E && part == 0) order[rank] = e;
        }
    }
    if (keep) {
#pragma unroll
        for (int i = 0; i < KEEP; ++i) {
            const int pr = tid + i * nt;
            const int e = mine[i], t = pr / topk;
            if (e < 0 || e >= E) continue;
            const uint32_t word = bm[e * W + (t >> 5)];
            const int pos = seg[e] + (int)pre[e * W + (t >> 5)] + __popc(word & ((1u << (t & 31)) - 1u));
            perm[pos] = pr;
        }
    } else {
        for (int pr = tid; pr < P; pr += nt) {
            const int e = idx[pr], t = pr / topk;
            if (e < 0 || e >= E) continue;
            const uint32_t word = bm[e * W + (t >> 5)];
            const int pos = seg[e] + (int)pre[e * W + (t >> 5)] + __popc(word & ((1u << (t & 31)) - 1u));
            perm[pos] = pr;
        }
    }
}

// ------------------------------------------------------- a11 grouped GEMMs
// One kernel for both expert contractions.  A workgroup of 4 waves owns two groups of 16 weight rows of one
// expert (gate/up: rows n0.. of wg and the same rows of wu, so SwiGLU happens in the epilogue; down: rows
// n0.. and n0+16.. of wd) and walks the expert's tokens 32 at a time.  Waves split K.  Every wave streams
// its K slice through a private ring of LDS stages filled by direct-to-LDS loads of 8 rows x 128 bytes
// (weights and gathered activation rows alike; a load shaped like an MFMA fragment, 16 rows x 64 bytes, runs
// at a third of the bandwidth), XOR-swizzled so that the v_mfma_i32_16x16x64_i8 fragment reads are conflict
// free.  No barrier inside the stream; partial accumulators of the four waves meet in LDS.
typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;
template <int N>
__device__ __forceinline__ void wait_vm()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

constexpr int MT = 2;             // 16-token fragments per pass
constexpr int NGRP = 2;           // 16-row weight groups per workgroup
constexpr int RING = 2;           // stages per wave
constexpr int BLK = 2 * (NGRP + MT);
constexpr int STAGE_BYTES = BLK * 1024;
constexpr int RING_BYTES = 4 * RING * STAGE_BYTES;
constexpr int EXPERT_LDS = RING_BYTES + 4 * NGRP * MT * 4 * 64 * 4;

template <bool DOWN>
__global__ __launch_bounds__(256) void k_moe_expert_gemm(const int8_t *__restrict__ act,
                                                         const float *__restrict__ act_scale,
                                                         const int32_t *__restrict__ perm,
                                                         const int32_t *__restrict__ seg_off,
                                                         const int8_t *__restrict__ w0, const float *__restrict__ sc0,
                                                         const int8_t *__restrict__ w1, const float *__restrict__ sc1,
                                                         float *__restrict__ out, int Kdim, int Nrows, int Hout,
                                                         int topk, int nch)
{
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int e = blockIdx.y;
    const int seg0 = seg_off[e], count = seg_off[e + 1] - seg0;
    if (count <= 0) return;
    // gate/up: the 4 waves split K (2048 bytes = 16 steps).  down: K is short (768 bytes = 6 steps), so each
    // wave takes its own 32 rows over the whole of K and nothing has to be added across waves
    // A workgroup walks `nch` consecutive row chunks (16 rows for gate/up, 128 for down) as ONE stream: the
    // loads of the next chunk are already in flight while the partial sums of this one are added and stored,
    // and the segment / permutation lookups are paid once per workgroup.
    constexpr int CHUNK_ROWS = DOWN ? 128 : 16;
    const int n0 = DOWN ? blockIdx.x * nch * 128 + wave * 32 : blockIdx.x * nch * 16;
    char *ring = smem + wave * (RING * STAGE_BYTES);
    int *s_part = reinterpret_cast<int *>(smem + RING_BYTES);   // [4 waves][NGRP][MT][4][64]

    // load side: lane l = 8*rho + c fetches chunk c ^ sigma(rho, block parity) of row rho of the block
    const int rho = lane >> 3, c8 = lane & 7;
    const int8_t *wsrc[2 * NGRP];
#pragma unroll
    for (int b = 0; b < 2 * NGRP; ++b) {
        const int sigma = ((b & 1) << 2) | (rho >> 1);
        const int grp = b >> 1;
        int rowi = n0 + (DOWN ? grp * 16 : 0) + (b & 1) * 8 + rho;
        if (rowi > Nrows - 1) rowi = Nrows - 1;
        const int8_t *base = (DOWN || grp == 0) ? w0 : w1;
        wsrc[b] = base + ((int64_t)e * Nrows + rowi) * Kdim + ((c8 ^ sigma) << 4);
    }
    const int steps = Kdim >> 7;
    const int s0 = DOWN ? 0 : steps * wave / 4, s1 = DOWN ? steps : steps * (wave + 1) / 4;

    // read side: fragment (16-row group, K half kk): lane (r = l%16, g = l/16) reads row r, chunk 4*kk + g
    const int r = lane & 15, g_ = lane >> 4;
    int roff[2];
    {
        const int rr = r & 7, bpar = r >> 3;
        const int sigma = (bpar << 2) | (rr >> 1);
        roff[0] = bpar * 1024 + ((8 * rr + ((0 + g_) ^ sigma)) << 4);
        roff[1] = bpar * 1024 + ((8 * rr + ((4 + g_) ^ sigma)) << 4);
    }

    for (int base = 0; base < count; base += 16 * MT) {
        // gathered activation rows of this pass (rows past the segment repeat its last row and are never stored)
        const int8_t *xsrc[2 * MT];
#pragma unroll
        for (int b = 0; b < 2 * MT; ++b) {
            const int sigma = ((b & 1) << 2) | (rho >> 1);
            const int pos = seg0 + min(base + b * 8 + rho, count - 1);
            const int64_t arow = DOWN ? (int64_t)pos : (int64_t)(perm[pos] / topk);
            xsrc[b] = act + arow * Kdim + ((c8 ^ sigma) << 4);
        }
        const int nsw = s1 - s0;            // K steps of this wave per chunk
        const int total_f = nch * nsw;      // flattened (chunk, step) stages of this wave
        auto issue = [&](int slot, int f) {
            const int fc = f < total_f ? f : total_f - 1;   // past the end: re-fetch the last stage (uniform vmcnt arithmetic)
            const int ch = fc / nsw, st = s0 + (fc - ch * nsw);
            char *sb = ring + slot * STAGE_BYTES;
            const int64_t koff = (int64_t)st * 128;
            const int64_t woff = (int64_t)ch * CHUNK_ROWS * Kdim + koff;
#pragma unroll
            for (int b = 0; b < 2 * NGRP; ++b)
                __builtin_amdgcn_global_load_lds((gptr_t)(wsrc[b] + woff), (lptr_t)(sb + b * 1024), 16, 0, 0);
#pragma unroll
            for (int b = 0; b < 2 * MT; ++b)
                __builtin_amdgcn_global_load_lds((gptr_t)(xsrc[b] + koff), (lptr_t)(sb + (2 * NGRP + b) * 1024), 16, 0, 0);
        };
        if (nsw > 0) {
#pragma unroll
            for (int d = 0; d < RING; ++d) issue(d, d);
        }
        int slot = 0, f = 0;
        for (int ch = 0; ch < nch; ++ch) {
        const int nc0 = n0 + ch * CHUNK_ROWS;
        v4i acc[NGRP][MT];
#pragma unroll
        for (int a = 0; a < NGRP; ++a)
#pragma unroll
            for (int b = 0; b < MT; ++b) acc[a][b] = (v4i){0, 0, 0, 0};
        for (int i = 0; i < nsw; ++i, ++f) {
            wait_vm<(RING - 1) * BLK>();   // the oldest stage in flight has landed
            const char *sb = ring + slot * STAGE_BYTES;
            v4i wf[NGRP][2], xf[MT][2];
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
                for (int a = 0; a < NGRP; ++a) wf[a][kk] = *reinterpret_cast<const v4i *>(sb + a * 2048 + roff[kk]);
#pragma unroll
                for (int b = 0; b < MT; ++b) xf[b][kk] = *reinterpret_cast<const v4i *>(sb + (NGRP + b) * 2048 + roff[kk]);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // fragments are in registers: the slot may be refilled
            issue(slot, f + RING);
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
#pragma unroll
                for (int a = 0; a < NGRP; ++a)
#pragma unroll
                    for (int b = 0; b < MT; ++b)
                        acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[a][kk], xf[b][kk], acc[a][b], 0, 0, 0);
            slot = slot + 1 == RING ? 0 : slot + 1;
        }
        __syncthreads();   // the previous chunk's epilogue has finished reading s_part
#pragma unroll
        for (int a = 0; a < NGRP; ++a)
#pragma unroll
            for (int b = 0; b < MT; ++b)
#pragma unroll
                for (int q = 0; q < 4; ++q) s_part[(((wave * NGRP + a) * MT + b) * 4 + q) * 64 + lane] = acc[a][b][q];
        __syncthreads();
        // accumulator layout: lane l, register q  <->  weight row 4*(l/16)+q, token l%16
        auto total = [&](int a, int row, int nn) {
            const int b = row >> 4, src = (nn >> 2) * 16 + (row & 15), q = nn & 3;
            int sum = 0;
#pragma unroll
            for (int wv = 0; wv < 4; ++wv) sum += s_part[(((wv * NGRP + a) * MT + b) * 4 + q) * 64 + src];
            return sum;
        };
        auto own = [&](int wv, int a, int row, int nn) {   // down: one wave's accumulator is already the total
            const int b = row >> 4, src = (nn >> 2) * 16 + (row & 15), q = nn & 3;
            return s_part[(((wv * NGRP + a) * MT + b) * 4 + q) * 64 + src];
        };
        if constexpr (!DOWN) {
            // 32 tokens x 16 channels, channel fastest; h = silu(g) * u in sorted-pair order
            for (int o = tid; o < 16 * MT * 16; o += 256) {
                const int nl = o & 15, row = o >> 4;
                if (base + row >= count || nc0 + nl >= Nrows) continue;
                const int pos = seg0 + base + row;
                const float sxt = act_scale[perm[pos] / topk];
                const float gv = ((float)total(0, row, nl) * sxt) * sc0[(int64_t)e * Nrows + nc0 + nl];
                const float uv = ((float)total(1, row, nl) * sxt) * sc1[(int64_t)e * Nrows + nc0 + nl];
                out[(int64_t)pos * Nrows + nc0 + nl] = (gv / (1.0f + expf(-gv))) * uv;
            }
        } else {
            // 32 tokens x 128 channels (32 per wave); out[pair] in pair order, channel fastest
            const int nbase = (blockIdx.x * nch + ch) * 128;
            for (int o = tid; o < 16 * MT * 128; o += 256) {
                const int nl = o & 127, row = o >> 7;
                if (base + row >= count || nbase + nl >= Nrows) continue;
                const int pos = seg0 + base + row;
                const int sum = own(nl >> 5, (nl >> 4) & 1, row, nl & 15);
                out[(int64_t)perm[pos] * Hout + nbase + nl] =
                    ((float)sum * act_scale[pos]) * sc0[(int64_t)e * Nrows + nbase + nl];
            }
        }
        }   // chunks
        wait_vm<0>();   // trailing re-fetches must not write LDS after the workgroup has gone
    }
}

// The same contraction with the activation fragments held in registers (possible when a wave's K slice is at
// most NSMAX steps of 128 bytes): only weights travel through the ring, twice as many of them are in flight
// for the same LDS, and a workgroup walks several row chunks against one set of activation registers.
// stages in flight per wave.  The down projection's workgroups are short (two chunks of 768-byte rows) and pay
// their set-up (segment -> permutation -> activation rows, two dependent round trips) for little streaming: a ring
// of two stages lets three of them share a compute unit instead of two (measured 61.5 -> 56 us); gate/up streams
// six chunks of 2048-byte rows per workgroup and is better off with four stages in flight.
constexpr int rx_ring(bool down) { return down ? 2 : 4; }
constexpr int RX_STAGE = 2 * NGRP * 1024;
constexpr int rx_ring_bytes(bool down) { return 4 * rx_ring(down) * RX_STAGE; }
constexpr int RX_MT = 3;   // most 16-token fragments per pass
constexpr int RX_RED_BYTES = NGRP * RX_MT * 4 * 64 * 4;
constexpr int rx_lds(bool down) { return rx_ring_bytes(down) + RX_RED_BYTES + 16 * RX_MT * 8 + 8 * 128 * 4; }   // + metadata + scales of <= 8 chunks

template <bool DOWN, int NSMAX, int MTT>
__device__ __forceinline__ void moe_expert_rx_body(const int8_t *__restrict__ act,
                                                         const float *__restrict__ act_scale,
                                                         const int32_t *__restrict__ perm,
                                                         const int32_t *__restrict__ seg_off,
                                                         const int8_t *__restrict__ w0, const float *__restrict__ sc0,
                                                         const int8_t *__restrict__ w1, const float *__restrict__ sc1,
                                                         float *__restrict__ out, int Kdim, int Nrows, int Hout,
                                                         int topk, int nch, int e, int bx)
{
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int seg0 = seg_off[e], count = seg_off[e + 1] - seg0;
    if (count <= 0) return;
    // gate/up: the 4 waves split K (2048 bytes = 16 steps).  down: K is short (768 bytes = 6 steps), so each
    // wave takes its own 32 rows over the whole of K and nothing has to be added across waves
    // A workgroup walks `nch` consecutive row chunks (16 rows for gate/up, 128 for down) as ONE stream: the
    // loads of the next chunk are already in flight while the partial sums of this one are added and stored,
    // and the segment / permutation lookups are paid once per workgroup.
    constexpr int CHUNK_ROWS = DOWN ? 128 : 16;
    const int n0 = DOWN ? bx * nch * 128 + wave * 32 : bx * nch * 16;
    constexpr int RX_RING = rx_ring(DOWN), RX_RING_BYTES = rx_ring_bytes(DOWN);
    char *ring = smem + wave * (RX_RING * RX_STAGE);
    int *s_red = reinterpret_cast<int *>(smem + RX_RING_BYTES);    // [NGRP][MTT][4][64] sums over the four K slices (gate/up)
    // per-pass token metadata and per-chunk weight scales sit in LDS so that the epilogue of a chunk issues no
    // dependent global loads (each would cost a memory round trip per chunk)
    int *s_dst = reinterpret_cast<int *>(smem + RX_RING_BYTES + RX_RED_BYTES);                  // [16*MTT] output row
    float *s_tsc = reinterpret_cast<float *>(s_dst + 16 * MTT);                                  // [16*MTT] token scale
    float *s_wsc = s_tsc + 16 * MTT;                                                             // [nch][SCW]
    constexpr int SCW = DOWN ? 128 : 32;
    // weight scales of every chunk: requested here, parked in LDS only after the weight stream and the
    // activation loads have been issued, so that the whole set-up costs one memory round trip
    float wsv[4];   // nch * SCW <= 8 * 128 = 4 values per thread
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int o = tid + u * 256;
        const int ch = o / SCW, nl = o - ch * SCW;
        float v = 0.0f;
        if (o < nch * SCW) {
            if constexpr (DOWN) {
                const int n = (bx * nch + ch) * 128 + nl;
                if (n < Nrows) v = sc0[(int64_t)e * Nrows + n];
            } else {
                const int n = (bx * nch + ch) * 16 + (nl & 15);
                if (n < Nrows) v = (nl < 16 ? sc0 : sc1)[(int64_t)e * Nrows + n];
            }
        }
        wsv[u] = v;
    }
    if constexpr (!DOWN) {
        for (int o = tid; o < NGRP * MTT * 256; o += 256) s_red[o] = 0;
    }

    // load side: lane l = 8*rho + c fetches chunk c ^ sigma(rho, block parity) of row rho of the block
    const int rho = lane >> 3, c8 = lane & 7;
    const int8_t *wsrc[2 * NGRP];
#pragma unroll
    for (int b = 0; b < 2 * NGRP; ++b) {
        const int sigma = ((b & 1) << 2) | (rho >> 1);
        const int grp = b >> 1;
        int rowi = n0 + (DOWN ? grp * 16 : 0) + (b & 1) * 8 + rho;
        if (rowi > Nrows - 1) rowi = Nrows - 1;
        const int8_t *base = (DOWN || grp == 0) ? w0 : w1;
        wsrc[b] = base + ((int64_t)e * Nrows + rowi) * Kdim + ((c8 ^ sigma) << 4);
    }
    const int steps = Kdim >> 7;
    const int s0 = DOWN ? 0 : steps * wave / 4, s1 = DOWN ? steps : steps * (wave + 1) / 4;

    // read side: fragment (16-row group, K half kk): lane (r = l%16, g = l/16) reads row r, chunk 4*kk + g
    const int r = lane & 15, g_ = lane >> 4;
    int roff[2];
    {
        const int rr = r & 7, bpar = r >> 3;
        const int sigma = (bpar << 2) | (rr >> 1);
        roff[0] = bpar * 1024 + ((8 * rr + ((0 + g_) ^ sigma)) << 4);
        roff[1] = bpar * 1024 + ((8 * rr + ((4 + g_) ^ sigma)) << 4);
    }

    for (int base = 0; base < count; base += 16 * MTT) {
        const int nsw = s1 - s0;            // K steps of this wave per chunk (<= NSMAX)
        const int total_f = nch * nsw;      // flattened (chunk, step) stages of this wave
        auto issue = [&](int slot, int f) {
            const int fc = f < total_f ? f : total_f - 1;   // past the end: re-fetch the last stage (uniform vmcnt arithmetic)
            const int ch = fc / nsw, st = s0 + (fc - ch * nsw);
            char *sb = ring + slot * RX_STAGE;
            const int64_t woff = (int64_t)ch * CHUNK_ROWS * Kdim + (int64_t)st * 128;
#pragma unroll
            for (int b = 0; b < 2 * NGRP; ++b)
                __builtin_amdgcn_global_load_lds((gptr_t)(wsrc[b] + woff), (lptr_t)(sb + b * 1024), 16, 0, 0);
        };
        // Activation rows of this pass, as MFMA fragments held in registers for every row chunk the workgroup
        // walks: lane (token r, 16-byte chunk g_ (+4)).  Rows past the segment repeat its last row and are never
        // stored.
        v4i xr[MTT][NSMAX][2];
        __syncthreads();   // the previous pass has finished with the token metadata and every ring is idle
        int m_dst = 0, m_pr = 0;
        if (tid < 16 * MTT && base + tid < count) {
            const int pos = seg0 + base + tid;
            m_pr = perm[pos];
            m_dst = DOWN ? m_pr : pos;
        }
        {
            // the weight stream starts first: its addresses do not depend on the tokens, whose lookups cost two
            // dependent memory round trips
            if (nsw > 0) {
#pragma unroll
                for (int d = 0; d < RX_RING; ++d) issue(d, d);
            }
#pragma unroll
            for (int b = 0; b < MTT; ++b) {
                const int pos = seg0 + min(base + b * 16 + r, count - 1);
                const int8_t *xp = act + (DOWN ? (int64_t)pos : (int64_t)(perm[pos] / topk)) * Kdim + g_ * 16;
#pragma unroll
                for (int i = 0; i < NSMAX; ++i) {
                    const int st = min(s0 + i, steps - 1);
                    xr[b][i][0] = *reinterpret_cast<const v4i *>(xp + (int64_t)st * 128);
                    xr[b][i][1] = *reinterpret_cast<const v4i *>(xp + (int64_t)st * 128 + 64);
                }
            }
        }

        if (tid < 16 * MTT && base + tid < count) {
            s_dst[tid] = m_dst;
            s_tsc[tid] = act_scale[DOWN ? seg0 + base + tid : m_pr / topk];
        }
        if (base == 0) {
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (tid + u * 256 < nch * SCW) s_wsc[tid + u * 256] = wsv[u];
        }
        __syncthreads();   // token metadata, weight scales and the zeroed sums are visible to every wave
        int slot = 0, f = 0;
        for (int ch = 0; ch < nch; ++ch) {
        const int nc0 = n0 + ch * CHUNK_ROWS;
        v4i acc[NGRP][MTT];
#pragma unroll
        for (int a = 0; a < NGRP; ++a)
#pragma unroll
            for (int b = 0; b < MTT; ++b) acc[a][b] = (v4i){0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < NSMAX; ++i) {
            if (i < nsw) {
                wait_vm<(RX_RING - 1) * 2 * NGRP>();   // the oldest stage in flight has landed
                const char *sb = ring + slot * RX_STAGE;
                v4i wf[NGRP][2];
#pragma unroll
                for (int kk = 0; kk < 2; ++kk)
#pragma unroll
                    for (int a = 0; a < NGRP; ++a) wf[a][kk] = *reinterpret_cast<const v4i *>(sb + a * 2048 + roff[kk]);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // fragments are in registers: the slot may be refilled
                issue(slot, f + RX_RING);
#pragma unroll
                for (int kk = 0; kk < 2; ++kk)
#pragma unroll
                    for (int a = 0; a < NGRP; ++a)
#pragma unroll
                        for (int b = 0; b < MTT; ++b)
                            acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[a][kk], xr[b][i][kk], acc[a][b], 0, 0, 0);
                slot = slot + 1 == RX_RING ? 0 : slot + 1;
                ++f;
            }
        }
        const float *wsc = s_wsc + ch * SCW;
        // accumulator layout: lane l, register q  <->  weight row 4*(l/16)+q, token l%16
        if constexpr (!DOWN) {
            // the four K slices meet in LDS by integer atomic adds (exact, order-free); whoever reads a sum puts
            // the zero back for the next chunk
#pragma unroll
            for (int a = 0; a < NGRP; ++a)
#pragma unroll
                for (int b = 0; b < MTT; ++b)
#pragma unroll
                    for (int q = 0; q < 4; ++q) atomicAdd(&s_red[((a * MTT + b) * 4 + q) * 64 + lane], acc[a][b][q]);
            __syncthreads();
            // 16*MTT tokens x 16 channels, channel fastest; h = silu(g) * u in sorted-pair order
#pragma unroll
            for (int o = tid; o < 16 * MTT * 16; o += 256) {
                const int nl = o & 15, row = o >> 4;
                const int bq = (((row >> 4) * 4) + (nl & 3)) * 64 + (nl >> 2) * 16 + (row & 15);
                const int gi = s_red[bq], ui = s_red[MTT * 256 + bq];
                s_red[bq] = 0;
                s_red[MTT * 256 + bq] = 0;
                if (base + row < count && nc0 + nl < Nrows) {
                    const float sxt = s_tsc[row];
                    const float gv = ((float)gi * sxt) * wsc[nl];
                    const float uv = ((float)ui * sxt) * wsc[16 + nl];
                    out[(int64_t)s_dst[row] * Nrows + nc0 + nl] = (gv / (1.0f + expf(-gv))) * uv;
                }
            }
            __syncthreads();   // the zeroes are in place before the next chunk's sums arrive
        } else {
            // every wave owns its 32 rows over the whole of K: results leave straight from the accumulators, four
            // consecutive channels of one token per lane; out[pair] in pair order
            const int nbase = (bx * nch + ch) * 128;
#pragma unroll
            for (int a = 0; a < NGRP; ++a) {
                const int nl = wave * 32 + a * 16 + 4 * g_;
                const float4 ws = *reinterpret_cast<const float4 *>(wsc + nl);
#pragma unroll
                for (int b = 0; b < MTT; ++b) {
                    const int row = b * 16 + r;
                    if (base + row < count && nbase + nl < Nrows) {
                        const float ts = s_tsc[row];
                        float4 o;
                        o.x = ((float)acc[a][b][0] * ts) * ws.x;
                        o.y = ((float)acc[a][b][1] * ts) * ws.y;
                        o.z = ((float)acc[a][b][2] * ts) * ws.z;
                        o.w = ((float)acc[a][b][3] * ts) * ws.w;
                        *reinterpret_cast<float4 *>(out + (int64_t)s_dst[row] * Hout + nbase + nl) = o;
                    }
                }
            }
        }
        }   // chunks
        wait_vm<0>();   // trailing re-fetches must not write LDS after the workgroup has gone
    }
}

// Grid: one dimension.  The first y_split experts of the size order are cut into workgroups of `nch` row chunks,
// the rest (the smallest segments, which run last: the launcher takes the last eighth) into workgroups of nch / 2
// chunks: the work that is left when the kernel runs dry then comes in pieces half as long, and the tail of the
// kernel with them (cfg4: 210 -> 205 us for the layer; halving a quarter or more of the experts gives it back).
template <bool DOWN, int NSMAX>
__global__ __launch_bounds__(256) void k_moe_expert_rx(const int8_t *__restrict__ act,
                                                       const float *__restrict__ act_scale,
                                                       const int32_t *__restrict__ perm,
                                                       const int32_t *__restrict__ seg_off,
                                                       const int8_t *__restrict__ w0, const float *__restrict__ sc0,
                                                       const int8_t *__restrict__ w1, const float *__restrict__ sc1,
                                                       float *__restrict__ out, int Kdim, int Nrows, int Hout,
                                                       int topk, int nch, const int32_t *__restrict__ order,
                                                       int chunks, int y_split)
{
    // workgroups are handed out in grid order: the experts with the most tokens go first
    const int wpe = (chunks + nch - 1) / nch;
    int y, bx, nchl;
    {
        const int i = blockIdx.x;
        if (i < y_split * wpe) {
            y = i / wpe; bx = i - y * wpe; nchl = nch;
        } else {
            nchl = nch > 1 ? nch / 2 : 1;
            const int wpe2 = (chunks + nchl - 1) / nchl;
            const int j = i - y_split * wpe;
            y = y_split + j / wpe2; bx = j - (j / wpe2) * wpe2;
        }
    }
    const int e = order[y];
    // tokens per pass follow the size of the expert's segment: every extra pass streams the weights again
    const int count = seg_off[e + 1] - seg_off[e];
    if (count <= 16)
        moe_expert_rx_body<DOWN, NSMAX, 1>(act, act_scale, perm, seg_off, w0, sc0, w1, sc1, out, Kdim, Nrows, Hout, topk, nchl, e, bx);
    else if (count <= 32 || NSMAX > 6)
        moe_expert_rx_body<DOWN, NSMAX, 2>(act, act_scale, perm, seg_off, w0, sc0, w1, sc1, out, Kdim, Nrows, Hout, topk, nchl, e, bx);
    else
        moe_expert_rx_body<DOWN, NSMAX, 3>(act, act_scale, perm, seg_off, w0, sc0, w1, sc1, out, Kdim, Nrows, Hout, topk, nchl, e, bx);
}

// y[t, n] = sum over slots in order of w[t, slot] * out[t*topk + slot, n].  A slot whose expert index lies outside
// [0, E) was never dispatched, so its row of `out` was never written: it contributes nothing.
// TOPK > 0: the slot count is known at compile time (the loads of a token are then all in flight at once); 0: any.
template <int TOPK>
__global__ __launch_bounds__(256) void k_moe_combine(const float *__restrict__ out, const float *__restrict__ w,
                                                     const int32_t *__restrict__ idx, float *__restrict__ y, int T,
                                                     int H, int topk_rt, int E)
{
    constexpr int NS = TOPK > 0 ? TOPK : MAX_TOPK;
    const int topk = TOPK > 0 ? TOPK : topk_rt;
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= (int64_t)T * H) return;
    const int t = (int)(i / H), n = (int)(i - (int64_t)t * H);
    // every load of the token goes out before the first use; a slot that was never dispatched is read like the
    // others (its row of the workspace exists, whatever it holds) and dropped by value
    float ws[NS];
    float4 v[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const int sc = s < topk ? s : topk - 1;
        const int e = idx[(int64_t)t * topk + sc];
        const bool ok = s < topk && e >= 0 && e < E;
        ws[s] = w[(int64_t)t * topk + sc];
        v[s] = *reinterpret_cast<const float4 *>(out + ((int64_t)t * topk + sc) * H + n);
        if (!ok) { ws[s] = 0.0f; v[s] = make_float4(0.f, 0.f, 0.f, 0.f); }
    }
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        if (s < topk) {
            a.x = a.x + ws[s] * v[s].x; a.y = a.y + ws[s] * v[s].y; a.z = a.z + ws[s] * v[s].z; a.w = a.w + ws[s] * v[s].w;
        }
    }
    *reinterpret_cast<float4 *>(y + i) = a;
}

struct Layout {
    int64_t off[11];
    int64_t total;
};

static Layout layout(int64_t T, int64_t H, int64_t I, int64_t E, int64_t topk)
{
    const int64_t P = T * topk;
    const int64_t sz[11] = {T * H, T * 4, P * 4, (2 * E + 1) * 4 /* seg_off, then experts by size */, P * I * 4, P * I, P * 4, P * H * 4, P * 4, P * 4, T * E * 4};
    Layout L;
    int64_t o = 0;
    for (int i = 0; i < 11; ++i) { L.off[i] = o; o += align_up(sz[i], 256); }
    L.total = o;
    return L;
}

static int32_t check_shapes(int64_t T, int64_t H, int64_t I, int64_t E, int32_t topk)
{
    if (T < 0 || H <= 0 || I <= 0 || E <= 0 || topk <= 0) return MI_EINVAL;   // T == 0: an empty batch, a call that does nothing
    if (H % 128 || I % 256 || topk > MAX_TOPK || topk > E) return MI_EINVAL;
    if (H > 32768 || I > 32768 || T * topk > (1LL << 24) || E > 65535) return MI_ERANGE;
    if (2 * E * ((T + 31) / 32) + E + 1 > DISPATCH_MAX_WORDS) return MI_ERANGE;  // dispatch bitmap in LDS
    return MI_OK;
}

// can the router's first kernel also produce the FFN's activation codes? (block 128, a wave per row)
static bool route_can_quantize(int64_t H) { return H % 128 == 0 && H <= 2048; }

// logits + top-k; qx / sx non-null (and route_can_quantize(H)): the logits kernel also rotates and quantizes x
static int32_t launch_route(const float *x, const float *wr, int32_t *idx, float *w, int64_t T, int64_t H, int64_t E,
                            int32_t topk, float *logits, int8_t *qx, float *sx, void *stream)
{
    // eight experts a wave (twice the workgroups) while sixteen would leave at most two workgroups to a compute unit
    const bool narrow = (int64_t)((T + 15) / 16) * (E / 16) <= 2 * (int64_t)compute_units();
    const dim3 grid((unsigned)((T + 15) / 16), (unsigned)(E / (narrow ? 8 : 16)));
    const int cq = qx ? (int)((H / 8 + 63) / 64) : 0;
#define MI_LOGITS(CQ_)                                                                                                  \
    do {                                                                                                                \
        if (narrow)                                                                                                     \
            hipLaunchKernelGGL((k_moe_logits<CQ_, 8>), grid, dim3(256), 0, as_stream(stream), x, wr, logits, (int)T,    \
                               (int)H, (int)E, qx, sx);                                                                 \
        else                                                                                                            \
            hipLaunchKernelGGL((k_moe_logits<CQ_, 16>), grid, dim3(256), 0, as_stream(stream), x, wr, logits, (int)T,   \
                               (int)H, (int)E, qx, sx);                                                                 \
    } while (0)
    switch (cq) {
    case 0: MI_LOGITS(0); break;
    case 1: MI_LOGITS(1); break;
    case 2: MI_LOGITS(2); break;
    case 3: MI_LOGITS(3); break;
    default: MI_LOGITS(4); break;
    }
#undef MI_LOGITS
    int32_t rc = launch_status();
    if (rc) return rc;
    hipLaunchKernelGGL(k_moe_topk, dim3((unsigned)((T + 3) / 4)), dim3(256), 0, as_stream(stream), logits, idx, w, (int)T,
                       (int)E, (int)topk);
    return launch_status();
}

}  // namespace moe
}  // namespace mi

using namespace mi;

extern "C" int64_t mi_moe_route_workspace_bytes(int64_t T, int64_t E)
{
    if (T < 0 || E <= 0) return MI_EINVAL;
    return moe::align_up(T * E * 4, 256);
}

extern "C" int32_t mi_moe_route(const float *x, const float *wr, int32_t *idx, float *w, int64_t T, int64_t H,
                                int64_t E, int32_t topk, void *workspace, int64_t workspace_bytes, void *stream)
{
    if (!x || !wr || !idx || !w || T < 0 || H <= 0 || E <= 0 || topk <= 0) return MI_EINVAL;
    if (H % 256 || E % 16 || topk > moe::MAX_TOPK || topk > E) return MI_EINVAL;
    if (E > 256 || T > (1LL << 24)) return MI_ERANGE;
    if (!aligned16(x) || !aligned16(wr) || !aligned4(idx) || !aligned4(w)) return MI_EINVAL;
    if (!workspace || !aligned16(workspace)) return MI_EINVAL;
    if (workspace_bytes < mi_moe_route_workspace_bytes(T, E)) return MI_ENOSPC;
    if (T == 0) return MI_OK;
    return moe::launch_route(x, wr, idx, w, T, H, E, topk, static_cast<float *>(workspace), nullptr, nullptr, stream);
}

static int32_t launch_dispatch(const int32_t *idx, int32_t *perm, int32_t *seg_off, int32_t *order, int64_t T,
                               int64_t E, int32_t topk, void *stream)
{
    if (!idx || !perm || !seg_off || T < 0 || E <= 0 || topk <= 0) return MI_EINVAL;
    if (T * topk > (1LL << 24) || E > 65535) return MI_ERANGE;
    const int64_t words = 2 * E * ((T + 31) / 32) + E + 1;
    if (words > moe::DISPATCH_MAX_WORDS) return MI_ERANGE;
    MI_LDS_OPT_IN((&moe::k_moe_dispatch), (int)(moe::DISPATCH_MAX_WORDS * 4));
    hipLaunchKernelGGL(moe::k_moe_dispatch, dim3(1), dim3(1024), (size_t)words * 4, as_stream(stream), idx, perm,
                       seg_off, order, (int)T, (int)E, (int)topk);
    return launch_status();
}

extern "C" int32_t mi_moe_dispatch(const int32_t *idx, int32_t *perm, int32_t *seg_off, int64_t T, int64_t E,
                                   int32_t topk, void *stream)
{
    return launch_dispatch(idx, perm, seg_off, nullptr, T, E, topk, stream);
}

extern "C" int64_t mi_moe_ffn_workspace_bytes(int64_t T, int64_t H, int64_t I, int64_t E, int32_t topk)
{
    int32_t rc = moe::check_shapes(T, H, I, E, topk);
    if (rc) return rc;
    return moe::layout(T, H, I, E, topk).total;
}

extern "C" int64_t mi_moe_layer_workspace_bytes(int64_t T, int64_t H, int64_t I, int64_t E, int32_t topk)
{
    return mi_moe_ffn_workspace_bytes(T, H, I, E, topk);
}

extern "C" int64_t mi_moe_ffn_workspace_offset(int32_t which, int64_t T, int64_t H, int64_t I, int64_t E,
                                               int32_t topk)
{
    int32_t rc = moe::check_shapes(T, H, I, E, topk);
    if (rc) return rc;
    if (which < 0 || which > 10) return MI_EINVAL;
    return moe::layout(T, H, I, E, topk).off[which];
}

// codes_ready: the activation codes and scales already sit in the workspace (written by the router's first kernel)
static int32_t run_ffn(const float *x, const int32_t *idx, const float *w, const int8_t *wg, const float *sg,
                       const int8_t *wu, const float *su, const int8_t *wd, const float *sd, float *y, int64_t T,
                       int64_t H, int64_t I, int64_t E, int32_t topk, void *workspace, int64_t workspace_bytes,
                       void *stream, bool codes_ready)
{
    int32_t rc = moe::check_shapes(T, H, I, E, topk);
    if (rc) return rc;
    if (!x || !idx || !w || !wg || !sg || !wu || !su || !wd || !sd || !y || !workspace) return MI_EINVAL;
    if (!aligned16(x) || !aligned16(wg) || !aligned16(wu) || !aligned16(wd) || !aligned16(y) || !aligned16(workspace))
        return MI_EINVAL;
    const moe::Layout L = moe::layout(T, H, I, E, topk);
    if (workspace_bytes < L.total) return MI_ENOSPC;
    if (T == 0) return MI_OK;
    char *ws = static_cast<char *>(workspace);
    int8_t *qx = reinterpret_cast<int8_t *>(ws + L.off[0]);
    float *sx = reinterpret_cast<float *>(ws + L.off[1]);
    int32_t *perm = reinterpret_cast<int32_t *>(ws + L.off[2]);
    int32_t *seg = reinterpret_cast<int32_t *>(ws + L.off[3]);
    float *h = reinterpret_cast<float *>(ws + L.off[4]);
    int8_t *hq = reinterpret_cast<int8_t *>(ws + L.off[5]);
    float *hs = reinterpret_cast<float *>(ws + L.off[6]);
    float *out = reinterpret_cast<float *>(ws + L.off[7]);
    hipStream_t s = as_stream(stream);
    const int64_t P = T * topk;

    int32_t *order = seg + E + 1;
    rc = launch_dispatch(idx, perm, seg, order, T, E, topk, stream);
    if (rc) return rc;
    if (!codes_ready) {
        rc = mi_fwht_quant_f32_i8(x, qx, sx, T, H, 128, stream);
        if (rc) return rc;
    }
    MI_LDS_OPT_IN((&moe::k_moe_expert_gemm<false>), moe::EXPERT_LDS);
    MI_LDS_OPT_IN((&moe::k_moe_expert_gemm<true>), moe::EXPERT_LDS);
    // Row chunks per workgroup: with the activation fragments in registers a workgroup walks several chunks
    // against them; about four workgroups per compute unit keep the stream dense.
    const int cus = compute_units();
    auto pick_nch = [&](int64_t chunks) {
        int64_t n = chunks * E / (4LL * cus);
        return (int)(n < 1 ? 1 : (n > 8 ? 8 : n));
    };
    const int steps_gu = (int)(H / 128), ns_gu = (steps_gu + 3) / 4;   // K steps per wave (the four waves split K)
    if (ns_gu <= 8) {
        const int nch = pick_nch(I / 16);
        const int chunks = (int)(I / 16), y_split = (int)(E - E / 8);
        const int wpe = (chunks + nch - 1) / nch, nch2 = nch > 1 ? nch / 2 : 1, wpe2 = (chunks + nch2 - 1) / nch2;
        const dim3 grid((unsigned)(y_split * wpe + (E - y_split) * wpe2));
#define MI_RX_GU(NS)                                                                                            \
    do {                                                                                                        \
        MI_LDS_OPT_IN((&moe::k_moe_expert_rx<false, NS>), moe::rx_lds(false));                                        \
        hipLaunchKernelGGL((moe::k_moe_expert_rx<false, NS>), grid, dim3(256), moe::rx_lds(false), s, qx, sx, perm, seg, \
                           wg, sg, wu, su, h, (int)H, (int)I, (int)I, (int)topk, nch, order, chunks, y_split);  \
    } while (0)
        if (ns_gu <= 2) MI_RX_GU(2);
        else if (ns_gu <= 4) MI_RX_GU(4);
        else MI_RX_GU(8);
#undef MI_RX_GU
    } else {
        hipLaunchKernelGGL(moe::k_moe_expert_gemm<false>, dim3((unsigned)(I / 16), (unsigned)E), dim3(256),
                           moe::EXPERT_LDS, s, qx, sx, perm, seg, wg, sg, wu, su, h, (int)H, (int)I, (int)I, (int)topk,
                           1);
    }
    rc = launch_status();
    if (rc) return rc;
    rc = mi_fwht_quant_f32_i8(h, hq, hs, P, I, 256, stream);
    if (rc) return rc;
    const int steps_dn = (int)(I / 128);   // every wave walks the whole of K
    if (steps_dn <= 8) {
        const int chunks = (int)((H + 127) / 128);
        const int nch = pick_nch(chunks), y_split = (int)(E - E / 8);
        const int wpe = (chunks + nch - 1) / nch, nch2 = nch > 1 ? nch / 2 : 1, wpe2 = (chunks + nch2 - 1) / nch2;
        const dim3 grid((unsigned)(y_split * wpe + (E - y_split) * wpe2));
#define MI_RX_DN(NS)                                                                                            \
    do {                                                                                                        \
        MI_LDS_OPT_IN((&moe::k_moe_expert_rx<true, NS>), moe::rx_lds(true));                                        \
        hipLaunchKernelGGL((moe::k_moe_expert_rx<true, NS>), grid, dim3(256), moe::rx_lds(true), s, hq, hs, perm, seg, wd, \
                           sd, (const int8_t *)nullptr, (const float *)nullptr, out, (int)I, (int)H, (int)H,    \
                           (int)topk, nch, order, chunks, y_split);                                             \
    } while (0)
        if (steps_dn <= 2) MI_RX_DN(2);
        else if (steps_dn <= 4) MI_RX_DN(4);
        else if (steps_dn <= 6) MI_RX_DN(6);
        else MI_RX_DN(8);
#undef MI_RX_DN
    } else {
        hipLaunchKernelGGL(moe::k_moe_expert_gemm<true>, dim3((unsigned)((H + 127) / 128), (unsigned)E), dim3(256),
                           moe::EXPERT_LDS, s, hq, hs, perm, seg, wd, sd, (const int8_t *)nullptr,
                           (const float *)nullptr, out, (int)I, (int)H, (int)H, (int)topk, 1);
    }
    rc = launch_status();
    if (rc) return rc;
    const dim3 cgrid((unsigned)((T * H / 4 + 255) / 256));
#define MI_COMBINE(K_) hipLaunchKernelGGL(moe::k_moe_combine<K_>, cgrid, dim3(256), 0, s, out, w, idx, y, (int)T, (int)H, (int)topk, (int)E)
    switch (topk) {
    case 1: MI_COMBINE(1); break;
    case 2: MI_COMBINE(2); break;
    case 4: MI_COMBINE(4); break;
    case 8: MI_COMBINE(8); break;
    default: MI_COMBINE(0); break;
    }
#undef MI_COMBINE
    return launch_status();
}

extern "C" int32_t mi_moe_ffn(const float *x, const int32_t *idx, const float *w, const int8_t *wg, const float *sg,
                              const int8_t *wu, const float *su, const int8_t *wd, const float *sd, float *y,
                              int64_t T, int64_t H, int64_t I, int64_t E, int32_t topk, void *workspace,
                              int64_t workspace_bytes, void *stream)
{
    return run_ffn(x, idx, w, wg, sg, wu, su, wd, sd, y, T, H, I, E, topk, workspace, workspace_bytes, stream, false);
}

extern "C" int32_t mi_moe_layer(const float *x, const float *wr, const int8_t *wg, const float *sg, const int8_t *wu,
                                const float *su, const int8_t *wd, const float *sd, float *y, int64_t T, int64_t H,
                                int64_t I, int64_t E, int32_t topk, void *workspace, int64_t workspace_bytes,
                                void *stream)
{
    int32_t rc = moe::check_shapes(T, H, I, E, topk);
    if (rc) return rc;
    if (!workspace || !aligned16(workspace)) return MI_EINVAL;
    const moe::Layout L = moe::layout(T, H, I, E, topk);
    if (workspace_bytes < L.total) return MI_ENOSPC;
    if (T == 0) return MI_OK;
    char *ws = static_cast<char *>(workspace);
    int32_t *idx = reinterpret_cast<int32_t *>(ws + L.off[8]);
    float *w = reinterpret_cast<float *>(ws + L.off[9]);
    // the checks of mi_moe_route, which this call stands in for
    if (!x || !wr || H % 256 || E % 16 || E > 256 || !aligned16(x) || !aligned16(wr)) return MI_EINVAL;
    const bool fuse = moe::route_can_quantize(H);
    rc = moe::launch_route(x, wr, idx, w, T, H, E, topk, reinterpret_cast<float *>(ws + L.off[10]),
                           fuse ? reinterpret_cast<int8_t *>(ws + L.off[0]) : nullptr,
                           fuse ? reinterpret_cast<float *>(ws + L.off[1]) : nullptr, stream);
    if (rc) return rc;
    return run_ffn(x, idx, w, wg, sg, wu, su, wd, sd, y, T, H, I, E, topk, workspace, workspace_bytes, stream, fuse);
}
