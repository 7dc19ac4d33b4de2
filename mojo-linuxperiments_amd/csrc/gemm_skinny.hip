// W8A8 contraction for skinny activations (decode GEMV, M <= 64):
//   acc[m,n] = sum_k qx[m,k] * qw[n,k],   y = ((float)acc * sx[m]) * sw[n]
// The weights [N,K] are read from HBM exactly once; everything else is small.
// Bound: HBM.  Algorithmic bytes per call = N*K (weights) + M*K (codes)
// + 4*M*N (output) + 4*(M+N) (scales).
//
// Kernels, chosen by M and K (launch_skinny):
//
//  k_gemv_reg (M = 1, and M <= 4 on K < 8192).  A lane always works on the same byte offsets of a weight row, so
//  its share of the activation codes lives in registers for the whole kernel: no LDS and no barrier in the
//  streaming part, 16 x 1 KB weight loads in flight per wave, v_dot4_i32_i8, one transposed butterfly per wave.
//  k_gemv_fused is the same kernel with the rotate + quantize prologue (and optionally the RMSNorm) inside, for
//  one token and K <= 4096.
//
//  k_gemv_dot4 (M <= 4, K that the register kernel cannot split evenly).  One workgroup per compute unit owns a
//  contiguous span of weight rows; the activation codes (M*K bytes) sit in LDS.  A wave streams one weight row
//  at a time with 128-bit loads, 1 KB contiguous per wave instruction, double buffered in registers, and each
//  lane feeds its 16 bytes to v_dot4_i32_i8 against the matching 16 bytes of every token.  The 64 partial int32
//  sums of a row meet in a DPP / swizzle wave reduction.  Exact: integer sums are order independent.
//
//  k_skinny_ring (4 < M <= 64, and M = 2..4 on K >= 8192).  v_mfma_i32_16x16x64_i8 wants 16 rows x 64
//  bytes per operand, but a load shaped like that touches 16 different lines
//  per quarter wave and runs at a third of the bandwidth of a load that takes
//  8 rows x 128 bytes.  So every wave owns a private ring of LDS stages, fills
//  it with direct-to-LDS loads of the good shape (weights and activation codes
//  alike, XOR-swizzled so that the fragment reads are conflict free) and reads
//  MFMA fragments back out.  The ring is private to the wave: no barrier in
//  the main loop, only vmcnt / lgkmcnt waits, and several stages stay in
//  flight per wave.  Waves of a workgroup split K; their partial accumulators
//  meet in LDS at the end.
#include <algorithm>
#include "common.h"
#include "fwht_core.h"

namespace mi {

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

// ------------------------------------------------------------------ M <= 4
__device__ __forceinline__ int wave_sum(int v)
{
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, true);   // quad_perm [1,0,3,2]
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
    v += __builtin_amdgcn_update_dpp(0, v, 0x124, 0xf, 0xf, true);  // row_ror:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x128, 0xf, 0xf, true);  // row_ror:8
    v += __builtin_amdgcn_ds_swizzle(v, 0x401F);                    // lane ^ 16
    v += __shfl_xor(v, 32, 64);
    return v;
}

// Transposed butterfly: `p` holds V (a power of two <= 64) per-lane partial sums; after the call lane l holds
// the wave-wide total of value  l >> (6 - log2 V)  (lanes that share those top bits hold the same total).
// Each round hands half of the values to the partner lane, so V values cost V - 1 shuffles + log-many, not 6 V.
template <int V, int OFF>
__device__ __forceinline__ void fold_sum(int (&p)[V], int lane)
{
    if constexpr (V > 1) {
        const bool hi = (lane & OFF) != 0;
        int q[V / 2];
#pragma unroll
        for (int i = 0; i < V / 2; ++i) {
            const int keep = hi ? p[i + V / 2] : p[i];
            const int send = hi ? p[i] : p[i + V / 2];
            q[i] = keep + __shfl_xor(send, OFF, 64);
        }
        fold_sum<V / 2, OFF / 2>(q, lane);
#pragma unroll
        for (int i = 0; i < V / 2; ++i) p[i] = q[i];
    } else {
#pragma unroll
        for (int off = OFF; off >= 1; off >>= 1) p[0] += __shfl_xor(p[0], off, 64);
    }
}

constexpr int pow2_ceil(int v) { int p = 1; while (p < v) p <<= 1; return p; }

// k_gemv_reg (M <= 4, K = 1024 * CW * QW up to a ragged last chunk): lane l always works on the same byte
// offsets of a row (16*l + 1024*c for the wave's CW chunks), so its share of the activation codes lives in
// registers for the whole kernel: no LDS, no barrier in the streaming part.  A wave issues all the loads of
// its R rows at once (R*CW <= 16 x 1 KB in flight per wave), runs v_dot4_i32_i8 on them and reduces its
// R*MB per-lane sums with one transposed butterfly.  QW waves that split a row add their totals in LDS.
template <int MB, int CW, bool DEQ>
__global__ __launch_bounds__(256) void k_gemv_reg(const int8_t *__restrict__ qx, const int8_t *__restrict__ qw,
                                                  const float *__restrict__ sx, const float *__restrict__ sw,
                                                  int32_t *__restrict__ acc_out, float *__restrict__ y, int M,
                                                  int N, int K, int QW)
{
    constexpr int R = (16 / CW) < 1 ? 1 : (16 / CW);   // rows per wave
    constexpr int V = pow2_ceil(R * MB);
    __shared__ int s_red[4][V];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q = wave % QW;                  // which CW-chunk slice of the row
    const int rows_per_wg = (4 / QW) * R;
    const int row0 = blockIdx.x * rows_per_wg + (wave / QW) * R;
    const int kbase = q * CW * 1024 + lane * 16;

    v4i w[R][CW];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int c = 0; c < CW; ++c) {
            const int off = kbase + c * 1024;
            w[r][c] = (row0 + r < N && off < K) ? *reinterpret_cast<const v4i *>(qw + (int64_t)(row0 + r) * K + off)
                                                : (v4i){0, 0, 0, 0};
        }
    v4i xr[MB][CW];
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int c = 0; c < CW; ++c) {
            const int off = kbase + c * 1024;
            const int ms = m < M ? m : M - 1;
            xr[m][c] = off < K ? *reinterpret_cast<const v4i *>(qx + (int64_t)ms * K + off) : (v4i){0, 0, 0, 0};
        }
    int p[V];
#pragma unroll
    for (int i = 0; i < V; ++i) p[i] = 0;
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            int a = 0;
#pragma unroll
            for (int c = 0; c < CW; ++c) {
                a = __builtin_amdgcn_sdot4(w[r][c][0], xr[m][c][0], a, false);
                a = __builtin_amdgcn_sdot4(w[r][c][1], xr[m][c][1], a, false);
                a = __builtin_amdgcn_sdot4(w[r][c][2], xr[m][c][2], a, false);
                a = __builtin_amdgcn_sdot4(w[r][c][3], xr[m][c][3], a, false);
            }
            p[r * MB + m] = a;
        }
    fold_sum<V, 32>(p, lane);
    // lane l holds value v = l >> SH; the first lane of each group of 64/V lanes speaks for it
    constexpr int SH = 6 - __builtin_ctz(V);
    const int v = lane >> SH;
    const bool speaker = (lane & ((1 << SH) - 1)) == 0;
    int total = p[0];
    if (QW > 1) {
        if (speaker) s_red[wave][v] = total;
        __syncthreads();
        if (q == 0 && speaker) {
            for (int o = 1; o < QW; ++o) total += s_red[wave + o][v];
        }
    }
    if (q == 0 && speaker && v < R * MB) {
        const int r = v / MB, m = v % MB, n = row0 + r;
        if (n < N && m < M) {
            if constexpr (DEQ) y[(int64_t)m * N + n] = ((float)total * sx[m]) * sw[n];
            else acc_out[(int64_t)m * N + n] = total;
        }
    }
}

// k_gemv_fused: k_gemv_reg with the rotate + quantize prologue inside.  The row's own loads go out first and the
// first group's weight loads right behind them; while the weights are in flight the workgroup rotates and quantizes
// the M activation rows (the same per-chunk code as the stand-alone quantizer, so the codes and scales are
// bit-identical), parks the codes in LDS and every lane picks up its share.  One launch per linear instead of two.
// ROT = false: the row arrives in the rotated basis and is only quantized.
// NORM: the row is first normalized, v = ((x (+ res)) * r) * g with r = 1 / sqrt(mean((x + res)^2) + eps), the
// arithmetic of the stand-alone RMSNorm + quantize kernel; workgroup 0 also leaves the residual sum (h_out) and, on
// request, the normalized row (xn_out) for the caller.
struct FusedNorm {
    const float *res, *g;
    float *h_out, *xn_out;
    float eps;
};

template <int MB, int CW, int CQ, bool NORM, bool ROT>
__global__ __launch_bounds__(256) void k_gemv_fused(const float *__restrict__ x, const int8_t *__restrict__ qw,
                                                    const float *__restrict__ sw, float *__restrict__ y,
                                                    int8_t *__restrict__ qx_out, float *__restrict__ sx_out, int M,
                                                    int N, int K, int QW, FusedNorm nm)
{
    constexpr int BLOCK = 128, LPB = BLOCK / 8;
    constexpr int R = (16 / CW) < 1 ? 1 : (16 / CW);   // rows per wave
    constexpr int V = pow2_ceil(R * MB);
    extern __shared__ __attribute__((aligned(16))) char s_dyn[];
    int8_t *s_x = reinterpret_cast<int8_t *>(s_dyn);                       // [MB][K] codes
    float *s_scale = reinterpret_cast<float *>(s_dyn + (size_t)MB * K);    // [MB]
    float *s_max = s_scale + MB;                                           // [4] row maxima, then [4 * CQ] sums of squares
    int *s_red = reinterpret_cast<int *>(s_max + 4 + 4 * CQ);              // [4][V]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q = wave % QW;                  // which CW-chunk slice of the row
    const int rows_per_wg = (4 / QW) * R;
    // the workgroup owns a run of consecutive groups of rows_per_wg weight rows (the groups dealt out evenly over
    // the grid): one prologue serves them all
    const int ngroups = (N + rows_per_wg - 1) / rows_per_wg;
    const int g0 = (int)((int64_t)ngroups * blockIdx.x / gridDim.x);
    const int g1 = (int)((int64_t)ngroups * (blockIdx.x + 1) / gridDim.x);
    const int kbase = q * CW * 1024 + lane * 16;

    auto load_w = [&](v4i (&w)[R][CW], int g) {
        const int row0 = g * rows_per_wg + (wave / QW) * R;
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < CW; ++c) {
                const int off = kbase + c * 1024;
                w[r][c] = (row0 + r < N && off < K) ? *reinterpret_cast<const v4i *>(qw + (int64_t)(row0 + r) * K + off)
                                                    : (v4i){0, 0, 0, 0};
            }
    };
    // Loads return in the order they were issued: the first row's own loads (activations, residual, gain) go out
    // BEFORE the first group's weights, so that the prologue's arithmetic runs while the weights are on their way
    // (issued behind them, the row would arrive only after 64 KB of weights per workgroup, and nothing would be in
    // flight while the prologue computes).
    v4i w[R][CW];

    // rotate + quantize, one row at a time: thread t owns chunks t, t + 256, ... of the row
    const int j = tid % LPB;
    const int nchunk = K / 8;
    for (int m = 0; m < MB && m < M; ++m) {
        const float *xr = x + (int64_t)m * K;
        float v[CQ][8];
        int base[CQ];
#pragma unroll
        for (int i = 0; i < CQ; ++i) {
            const int c = tid + i * 256;
            base[i] = (c / LPB) * BLOCK + 4 * j;
            if (c < nchunk) {
                const float4 lo = *reinterpret_cast<const float4 *>(xr + base[i]);
                const float4 hi = *reinterpret_cast<const float4 *>(xr + base[i] + BLOCK / 2);
                v[i][0] = lo.x; v[i][1] = lo.y; v[i][2] = lo.z; v[i][3] = lo.w;
                v[i][4] = hi.x; v[i][5] = hi.y; v[i][6] = hi.z; v[i][7] = hi.w;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[i][e] = 0.0f;
            }
        }
        const bool keeper = blockIdx.x == 0;   // one workgroup also leaves the codes and scales in the caller's workspace
        if constexpr (!NORM) {
            if (m == 0) load_w(w, g0);
        }
        if constexpr (NORM) {
            float4 gl[CQ], gh[CQ], rl_[CQ], rh_[CQ];
            float ss[CQ];   // per chunk, then per group of 64 chunks (group wave + 4 * i): the order of fwht_core.h
#pragma unroll
            for (int i = 0; i < CQ; ++i) {
                if (tid + i * 256 < nchunk) {
                    gl[i] = *reinterpret_cast<const float4 *>(nm.g + base[i]);
                    gh[i] = *reinterpret_cast<const float4 *>(nm.g + base[i] + BLOCK / 2);
                    if (nm.res) {
                        const float *rr = nm.res + (int64_t)m * K + base[i];
                        rl_[i] = *reinterpret_cast<const float4 *>(rr);
                        rh_[i] = *reinterpret_cast<const float4 *>(rr + BLOCK / 2);
                    }
                }
            }
            if (m == 0) load_w(w, g0);
#pragma unroll
            for (int i = 0; i < CQ; ++i) {
                ss[i] = 0.0f;
                if (tid + i * 256 < nchunk) {
                    if (nm.res) {
                        const float4 rl = rl_[i], rh = rh_[i];
                        v[i][0] = v[i][0] + rl.x; v[i][1] = v[i][1] + rl.y; v[i][2] = v[i][2] + rl.z; v[i][3] = v[i][3] + rl.w;
                        v[i][4] = v[i][4] + rh.x; v[i][5] = v[i][5] + rh.y; v[i][6] = v[i][6] + rh.z; v[i][7] = v[i][7] + rh.w;
                        if (keeper) {
                            float *ho = nm.h_out + (int64_t)m * K + base[i];
                            *reinterpret_cast<float4 *>(ho) = make_float4(v[i][0], v[i][1], v[i][2], v[i][3]);
                            *reinterpret_cast<float4 *>(ho + BLOCK / 2) = make_float4(v[i][4], v[i][5], v[i][6], v[i][7]);
                        }
                    }
                    ss[i] = chunk_sumsq(v[i]);
                }
            }
#pragma unroll
            for (int i = 0; i < CQ; ++i) ss[i] = group_sum(ss[i]);
            __syncthreads();   // the previous row's sums have been read
            if (lane == 0) {
#pragma unroll
                for (int i = 0; i < CQ; ++i) s_max[4 + wave + 4 * i] = ss[i];
            }
            __syncthreads();
            const float total = tree_sum<4 * CQ>(s_max + 4);
            const float r = 1.0f / sqrtf(total / (float)K + nm.eps);
#pragma unroll
            for (int i = 0; i < CQ; ++i) {
                if (tid + i * 256 < nchunk) {
                    v[i][0] = (v[i][0] * r) * gl[i].x; v[i][1] = (v[i][1] * r) * gl[i].y;
                    v[i][2] = (v[i][2] * r) * gl[i].z; v[i][3] = (v[i][3] * r) * gl[i].w;
                    v[i][4] = (v[i][4] * r) * gh[i].x; v[i][5] = (v[i][5] * r) * gh[i].y;
                    v[i][6] = (v[i][6] * r) * gh[i].z; v[i][7] = (v[i][7] * r) * gh[i].w;
                    if (keeper && nm.xn_out) {
                        float *xo = nm.xn_out + (int64_t)m * K + base[i];
                        *reinterpret_cast<float4 *>(xo) = make_float4(v[i][0], v[i][1], v[i][2], v[i][3]);
                        *reinterpret_cast<float4 *>(xo + BLOCK / 2) = make_float4(v[i][4], v[i][5], v[i][6], v[i][7]);
                    }
                }
            }
        }
        float amax = 0.0f;
#pragma unroll
        for (int i = 0; i < CQ; ++i) {
            if constexpr (ROT) fwht_chunk<BLOCK>(v[i], j);   // !ROT: the row arrives in the rotated basis
            amax = fmaxf(amax, abs8(v[i]));
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
        __syncthreads();   // the previous row's maxima have been read
        if (lane == 0) s_max[wave] = amax;
        __syncthreads();
        const float a = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
        const float sc = (a == 0.0f) ? 1.0f : a / 127.0f;
        const float inv = (a == 0.0f) ? 0.0f : 127.0f / a;
        if (tid == 0) s_scale[m] = sc;
        int8_t *qrow = s_x + (size_t)m * K;
        if (keeper && tid == 0) sx_out[m] = sc;
#pragma unroll
        for (int i = 0; i < CQ; ++i) {
            if (tid + i * 256 < nchunk) {
                const uint32_t c0 = quant4(v[i][0], v[i][1], v[i][2], v[i][3], inv);
                const uint32_t c1 = quant4(v[i][4], v[i][5], v[i][6], v[i][7], inv);
                *reinterpret_cast<uint32_t *>(qrow + base[i]) = c0;
                *reinterpret_cast<uint32_t *>(qrow + base[i] + BLOCK / 2) = c1;
                if (keeper) {
                    *reinterpret_cast<uint32_t *>(qx_out + (int64_t)m * K + base[i]) = c0;
                    *reinterpret_cast<uint32_t *>(qx_out + (int64_t)m * K + base[i] + BLOCK / 2) = c1;
                }
            }
        }
    }
    __syncthreads();

    v4i xr[MB][CW];
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int c = 0; c < CW; ++c) {
            const int off = kbase + c * 1024;
            const int ms = m < M ? m : M - 1;
            xr[m][c] = off < K ? *reinterpret_cast<const v4i *>(s_x + (size_t)ms * K + off) : (v4i){0, 0, 0, 0};
        }
    constexpr int SH = 6 - __builtin_ctz(V);
    const int vi = lane >> SH;
    const bool speaker = (lane & ((1 << SH) - 1)) == 0;
#pragma unroll 1
    for (int g = g0; g < g1; ++g) {
        // the next group's weight loads go out before this group's arithmetic
        v4i wn[R][CW];
        const bool more = g + 1 < g1;   // the same for every thread of the workgroup
        if (more) load_w(wn, g + 1);
        int p[V];
#pragma unroll
        for (int i = 0; i < V; ++i) p[i] = 0;
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                int a = 0;
#pragma unroll
                for (int c = 0; c < CW; ++c) {
                    a = __builtin_amdgcn_sdot4(w[r][c][0], xr[m][c][0], a, false);
                    a = __builtin_amdgcn_sdot4(w[r][c][1], xr[m][c][1], a, false);
                    a = __builtin_amdgcn_sdot4(w[r][c][2], xr[m][c][2], a, false);
                    a = __builtin_amdgcn_sdot4(w[r][c][3], xr[m][c][3], a, false);
                }
                p[r * MB + m] = a;
            }
        fold_sum<V, 32>(p, lane);
        int total = p[0];
        if (QW > 1) {
            if (speaker) s_red[wave * V + vi] = total;
            __syncthreads();
            if (q == 0 && speaker) {
                for (int o = 1; o < QW; ++o) total += s_red[(wave + o) * V + vi];
            }
            __syncthreads();   // s_red is free for the next group
        }
        if (q == 0 && speaker && vi < R * MB) {
            const int r = vi / MB, m = vi % MB, n = g * rows_per_wg + (wave / QW) * R + r;
            if (n < N && m < M) y[(int64_t)m * N + n] = ((float)total * s_scale[m]) * sw[n];
        }
        if (more) {
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int c = 0; c < CW; ++c) w[r][c] = wn[r][c];
        }
    }
}

template <int MB, int CW, int CQ, bool NORM, bool ROT = true>
static int32_t launch_fused(const float *x, const int8_t *qw, const float *sw, float *y, int8_t *qx, float *sx, int M,
                            int N, int K, int QW, const FusedNorm &nm, hipStream_t s)
{
    constexpr int R = (16 / CW) < 1 ? 1 : (16 / CW);
    constexpr int V = pow2_ceil(R * MB);
    const size_t lds = (size_t)MB * K + (MB + 4 + 4 * CQ) * sizeof(float) + 4 * V * sizeof(int);
    MI_LDS_OPT_IN((&k_gemv_fused<MB, CW, CQ, NORM, ROT>), 96 * 1024);
    // Every workgroup reads the whole activation row (with the norm: the residual and the gain too, 48 KB at
    // K = 4096) before its first dot product.  Beyond two workgroups per compute unit a workgroup therefore takes
    // several groups of rows in turn, the next group's weights on their way while it works on the current one.
    const int rows_per_wg = (4 / QW) * R;
    const int ngroups = (N + rows_per_wg - 1) / rows_per_wg;
    const unsigned grid = (unsigned)std::min(ngroups, 2 * compute_units());   // three per unit measured the same
    hipLaunchKernelGGL((k_gemv_fused<MB, CW, CQ, NORM, ROT>), dim3(grid), dim3(256), lds, s, x, qw, sw, y, qx, sx, M, N,
                       K, QW, nm);
    return launch_status();
}

// The fused decode linear is taken for one token and K <= 4096 only (MI_EINVAL tells the caller to take the
// two-kernel path).  Measured: 9.3 against 10.6 us for 4096 -> 6144 at M = 1, but every workgroup repeats the
// quantization, which at M = 4 or K = 14336 costs more than the launch it saves (15.6 against 11.7 us, 20.8
// against 18.8 us).  rotate = false: x is already in the rotated basis (the attention output as the merge leaves
// it) and is only quantized.
int32_t launch_linear_fused(const float *x, const int8_t *qw, const float *sw, float *y, int8_t *qx, float *sx,
                            int64_t M64, int64_t N64, int64_t K64, hipStream_t s, bool rotate)
{
    const int M = (int)M64, N = (int)N64, K = (int)K64;
    if (M != 1 || K % 1024) return MI_EINVAL;
    const int nchunk = K >> 10;
    const FusedNorm none = {nullptr, nullptr, nullptr, nullptr, 0.0f};
    if (rotate) {
        if (nchunk == 4) return launch_fused<1, 4, 2, false>(x, qw, sw, y, qx, sx, M, N, K, 1, none, s);   // K = 4096
        if (nchunk == 2) return launch_fused<1, 2, 1, false>(x, qw, sw, y, qx, sx, M, N, K, 1, none, s);   // K = 2048
    } else {
        if (nchunk == 4) return launch_fused<1, 4, 2, false, false>(x, qw, sw, y, qx, sx, M, N, K, 1, none, s);
        if (nchunk == 2) return launch_fused<1, 2, 1, false, false>(x, qw, sw, y, qx, sx, M, N, K, 1, none, s);
    }
    return MI_EINVAL;
}

// The same with the (residual +) RMSNorm ahead of the quantizer: one launch for norm + quantize + GEMV of one token.
int32_t launch_norm_linear_fused(const float *x, const float *res, const float *g, float eps, float *h_out,
                                 float *xn_out, const int8_t *qw, const float *sw, float *y, int8_t *qx, float *sx,
                                 int64_t M64, int64_t N64, int64_t K64, hipStream_t s)
{
    const int M = (int)M64, N = (int)N64, K = (int)K64;
    if (M != 1 || K % 1024) return MI_EINVAL;
    const int nchunk = K >> 10;
    const FusedNorm nm = {res, g, h_out, xn_out, eps};
    if (nchunk == 4) return launch_fused<1, 4, 2, true>(x, qw, sw, y, qx, sx, M, N, K, 1, nm, s);
    if (nchunk == 2) return launch_fused<1, 2, 1, true>(x, qw, sw, y, qx, sx, M, N, K, 1, nm, s);
    return MI_EINVAL;
}

template <int MB, bool DEQ>
__global__ __launch_bounds__(512) void k_gemv_dot4(const int8_t *__restrict__ qx, const int8_t *__restrict__ qw,
                                                   const float *__restrict__ sx, const float *__restrict__ sw,
                                                   int32_t *__restrict__ acc_out, float *__restrict__ y, int M,
                                                   int N, int K)
{
    extern __shared__ __attribute__((aligned(16))) char s_x[];  // [MB][K] activation codes
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwave = blockDim.x >> 6;
    const int n_lo = (int)((int64_t)N * blockIdx.x / gridDim.x), n_hi = (int)((int64_t)N * (blockIdx.x + 1) / gridDim.x);
    const int nchunk = (K + 1023) >> 10;   // 1 KB chunks per row; K % 128 == 0 so a chunk is whole for lane*16 < K - c*1024
    constexpr int U = 4;                   // loads in flight per buffer

    auto load_chunks = [&](v4i (&buf)[U], int row, int c0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int off = (c0 + u) * 1024 + lane * 16;
            buf[u] = (row < n_hi && off < K) ? *reinterpret_cast<const v4i *>(qw + (int64_t)row * K + off) : (v4i){0, 0, 0, 0};
        }
    };
    // first weight loads go out before the activation codes are staged
    v4i buf[2][U];
    int row = n_lo + wave, c0 = 0;
    load_chunks(buf[0], row, 0);

    for (int i = tid * 16; i < MB * K; i += blockDim.x * 16) {
        const int m = i / K, k = i - m * K;
        const int ms = m < M ? m : M - 1;   // rows past M repeat the last token and are never stored
        *reinterpret_cast<v4i *>(s_x + i) = *reinterpret_cast<const v4i *>(qx + (int64_t)ms * K + k);
    }
    __syncthreads();

    int acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m] = 0;
    int cur = 0;
    while (row < n_hi) {
        // next batch of this row, or the first batch of the wave's next row
        int nrow = row, nc0 = c0 + U;
        if (nc0 >= nchunk) { nrow = row + nwave; nc0 = 0; }
        load_chunks(buf[cur ^ 1], nrow, nc0);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int off = (c0 + u) * 1024 + lane * 16;
            if (off < K) {
                const v4i w = buf[cur][u];
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    const v4i xv = *reinterpret_cast<const v4i *>(s_x + m * K + off);
                    int a = acc[m];
                    a = __builtin_amdgcn_sdot4(w[0], xv[0], a, false);
                    a = __builtin_amdgcn_sdot4(w[1], xv[1], a, false);
                    a = __builtin_amdgcn_sdot4(w[2], xv[2], a, false);
                    a = __builtin_amdgcn_sdot4(w[3], xv[3], a, false);
                    acc[m] = a;
                }
            }
        }
        if (nrow != row) {
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                const int sum = wave_sum(acc[m]);
                if (lane == 0 && m < M) {
                    if constexpr (DEQ) y[(int64_t)m * N + row] = ((float)sum * sx[m]) * sw[row];
                    else acc_out[(int64_t)m * N + row] = sum;
                }
                acc[m] = 0;
            }
        }
        row = nrow;
        c0 = nc0;
        cur ^= 1;
    }
}

// --------------------------------------------------------------- 4 < M <= 64
template <int N>
__device__ __forceinline__ void wait_vm()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// NB blocks of 8 weight rows per workgroup, MT groups of 16 tokens, ring of D stages per wave.
// A stage = one 128-byte K step of (8*NB weight rows + 16*MT token rows) as 1 KB blocks of 8 rows.  The matrix
// instruction takes 16 weight rows: with NB odd the last group's second half reads whatever block follows (the first
// token block) and its 8 result rows are never stored.  8-row granularity lets the launcher give every compute
// unit the same number of rows (N / 8 blocks over the units: 3 a unit for N = 6144, 7 for N = 14336).
template <int NB, int MT, int D, bool DEQ>
__device__ __forceinline__ void ring_body(const int8_t *__restrict__ qx, const int8_t *__restrict__ qw,
                                          const float *__restrict__ sx, const float *__restrict__ sw,
                                          int32_t *__restrict__ acc_out, float *__restrict__ y, int M, int N, int K,
                                          const int n0, char *smem)
{
    constexpr int NG = (NB + 1) / 2;         // 16-row groups the matrix instructions work on
    constexpr int BLK = NB + 2 * MT;         // 1 KB blocks (= load instructions) per stage
    constexpr int STAGE = BLK * 1024;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), nwave = blockDim.x >> 6;
    char *ring = smem + wave * (D * STAGE);

    // load side: lane l = 8*rho + c fetches chunk c ^ sigma of row rho of the block
    const int8_t *src[BLK];
    {
        const int rho = lane >> 3, c = lane & 7;
#pragma unroll
        for (int b = 0; b < BLK; ++b) {
            // (the swizzle goes by the block's place in its own 16-row group: weight blocks and token blocks count apart)
            const int sigma = ((((b < NB) ? b : b - NB) & 1) << 2) | (rho >> 1);
            const int8_t *base;
            if (b < NB) {
                int rowi = n0 + b * 8 + rho;
                if (rowi > N - 1) rowi = N - 1;
                base = qw + (int64_t)rowi * K;
            } else {
                int tok = (b - NB) * 8 + rho;
                if (tok > M - 1) tok = M - 1;   // tokens past M repeat the last one and are never stored
                base = qx + (int64_t)tok * K;
            }
            src[b] = base + ((c ^ sigma) << 4);
        }
    }
    const int steps = K >> 7;
    const int s0 = (int)((int64_t)steps * wave / nwave), s1 = (int)((int64_t)steps * (wave + 1) / nwave);
    auto issue = [&](int slot, int s) {
        const int sc = s < s1 ? s : s1 - 1;   // past the slice: re-fetch the last step (keeps the vmcnt arithmetic uniform)
        char *sb = ring + slot * STAGE;
        const int64_t koff = (int64_t)sc * 128;
#pragma unroll
        for (int b = 0; b < BLK; ++b)
            __builtin_amdgcn_global_load_lds((gptr_t)(src[b] + koff), (lptr_t)(sb + b * 1024), 16, 0, 0);
    };

    // read side: fragment (16-row group t, K half kk): lane (r = l%16, g = l/16) reads row r, chunk 4*kk + g
    const int r = lane & 15, g_ = lane >> 4;
    int roff[2];
    {
        const int rho = r & 7, bpar = r >> 3;
        const int sigma = (bpar << 2) | (rho >> 1);
        roff[0] = bpar * 1024 + ((8 * rho + ((0 + g_) ^ sigma)) << 4);
        roff[1] = bpar * 1024 + ((8 * rho + ((4 + g_) ^ sigma)) << 4);
    }
    v4i acc[NG][MT];
#pragma unroll
    for (int a = 0; a < NG; ++a)
#pragma unroll
        for (int b = 0; b < MT; ++b) acc[a][b] = (v4i){0, 0, 0, 0};

    if (s1 > s0) {
#pragma unroll
        for (int d = 0; d < D; ++d) issue(d, s0 + d);
        int slot = 0;
        for (int s = s0; s < s1; ++s) {
            wait_vm<(D - 1) * BLK>();   // the oldest stage in flight has landed
            const char *sb = ring + slot * STAGE;
            v4i wf[NG][2], xf[MT][2];
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
                for (int a = 0; a < NG; ++a) wf[a][kk] = *reinterpret_cast<const v4i *>(sb + a * 2048 + roff[kk]);
#pragma unroll
                for (int b = 0; b < MT; ++b) xf[b][kk] = *reinterpret_cast<const v4i *>(sb + NB * 1024 + b * 2048 + roff[kk]);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // fragments are in registers: the slot may be refilled
            issue(slot, s + D);
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
#pragma unroll
                for (int a = 0; a < NG; ++a)
#pragma unroll
                    for (int b = 0; b < MT; ++b)
                        acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[a][kk], xf[b][kk], acc[a][b], 0, 0, 0);
            slot = slot + 1 == D ? 0 : slot + 1;
        }
        wait_vm<0>();   // nothing of this wave may still be writing LDS when the ring is reused below
    }
    __syncthreads();

    // partial accumulators of all waves -> LDS (the rings are idle now)
    int *s_part = reinterpret_cast<int *>(smem);   // [nwave][NG][MT][4][64]
#pragma unroll
    for (int a = 0; a < NG; ++a)
#pragma unroll
        for (int b = 0; b < MT; ++b)
#pragma unroll
            for (int e = 0; e < 4; ++e) s_part[(((wave * NG + a) * MT + b) * 4 + e) * 64 + lane] = acc[a][b][e];
    __syncthreads();
    // accumulator layout: lane l, register e  <->  weight row 4*(l/16)+e, token l%16
    for (int o = tid; o < 256 * NG * MT; o += blockDim.x) {
        const int nl = o % (16 * NG), m = o / (16 * NG);
        const int n = n0 + nl;
        if (m >= M || n >= N || nl >= 8 * NB) continue;
        const int a = nl >> 4, nn = nl & 15, b = m >> 4;
        const int src_lane = (nn >> 2) * 16 + (m & 15), e = nn & 3;
        int sum = 0;
        for (int w = 0; w < nwave; ++w) sum += s_part[(((w * NG + a) * MT + b) * 4 + e) * 64 + src_lane];
        if constexpr (DEQ) y[(int64_t)m * N + n] = ((float)sum * sx[m]) * sw[n];
        else acc_out[(int64_t)m * N + n] = sum;
    }
}

template <int NB, int MT, int D, bool DEQ>
__global__ __launch_bounds__(512) void k_skinny_ring(const int8_t *__restrict__ qx, const int8_t *__restrict__ qw,
                                                     const float *__restrict__ sx, const float *__restrict__ sw,
                                                     int32_t *__restrict__ acc_out, float *__restrict__ y, int M,
                                                     int N, int K)
{
    extern __shared__ __attribute__((aligned(16))) char smem[];
    ring_body<NB, MT, D, DEQ>(qx, qw, sx, sw, acc_out, y, M, N, K, (int)blockIdx.x * 8 * NB, smem);
}

// An odd number of 8-row blocks per compute unit, dealt to two workgroups of four waves that share the unit: the
// first half of the grid takes NBA blocks each, the second half NBB = NBA - 1 (the dispatcher fills every unit once
// before it places a second workgroup anywhere, so a unit gets one of each).
template <int NBA, int NBB, int MT, int D, bool DEQ>
__global__ __launch_bounds__(256) void k_skinny_ring_mixed(const int8_t *__restrict__ qx, const int8_t *__restrict__ qw,
                                                           const float *__restrict__ sx, const float *__restrict__ sw,
                                                           int32_t *__restrict__ acc_out, float *__restrict__ y, int M,
                                                           int N, int K)
{
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int half = (int)(gridDim.x >> 1), id = (int)blockIdx.x;
    if (id < half) ring_body<NBA, MT, D, DEQ>(qx, qw, sx, sw, acc_out, y, M, N, K, id * 8 * NBA, smem);
    else ring_body<NBB, MT, D, DEQ>(qx, qw, sx, sw, acc_out, y, M, N, K, half * 8 * NBA + (id - half) * 8 * NBB, smem);
}

template <int MB, bool DEQ>
static int32_t launch_dot4(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc,
                           float *y, int M, int N, int K, hipStream_t s)
{
    const size_t lds = (size_t)MB * K;
    MI_LDS_OPT_IN((&k_gemv_dot4<MB, DEQ>), 160 * 1024);
    const int cus = compute_units();
    // one or two workgroups per compute unit, each with a contiguous span of at least 8 rows
    int grid = lds <= 64 * 1024 ? 2 * cus : cus;
    if (grid > (N + 7) / 8) grid = (N + 7) / 8;
    hipLaunchKernelGGL((k_gemv_dot4<MB, DEQ>), dim3((unsigned)grid), dim3(512), lds, s, qx, qw, sx, sw, acc, y, M, N, K);
    return launch_status();
}

template <int MB, int CW, bool DEQ>
static int32_t launch_reg(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc,
                          float *y, int M, int N, int K, int QW, hipStream_t s)
{
    constexpr int R = (16 / CW) < 1 ? 1 : (16 / CW);
    const int rows_per_wg = (4 / QW) * R;
    const unsigned grid = (unsigned)((N + rows_per_wg - 1) / rows_per_wg);
    hipLaunchKernelGGL((k_gemv_reg<MB, CW, DEQ>), dim3(grid), dim3(256), 0, s, qx, qw, sx, sw, acc, y, M, N, K, QW);
    return launch_status();
}

template <int MB, bool DEQ>
static int32_t launch_reg_cw(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc,
                             float *y, int M, int N, int K, int CW, int QW, hipStream_t s)
{
    switch (CW) {
    case 1: return launch_reg<MB, 1, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, QW, s);
    case 2: return launch_reg<MB, 2, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, QW, s);
    case 3: return launch_reg<MB, 3, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, QW, s);
    case 4: return launch_reg<MB, 4, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, QW, s);
    case 5: return launch_reg<MB, 5, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, QW, s);
    case 6: return launch_reg<MB, 6, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, QW, s);
    default: return launch_reg<MB, 7, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, QW, s);
    }
}

template <int NB, int MT, int D, bool DEQ>
static int32_t launch_ring(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc,
                           float *y, int M, int N, int K, int nwave, hipStream_t s)
{
    constexpr int STAGE = (NB + 2 * MT) * 1024;
    constexpr int NG = (NB + 1) / 2;
    size_t lds = (size_t)nwave * D * STAGE;
    const size_t part = (size_t)nwave * NG * MT * 4 * 64 * sizeof(int);
    if (part > lds) lds = part;
    if (lds > 160 * 1024) return MI_ENOSPC;
    MI_LDS_OPT_IN((&k_skinny_ring<NB, MT, D, DEQ>), 160 * 1024);
    const unsigned grid = (unsigned)((N + 8 * NB - 1) / (8 * NB));
    hipLaunchKernelGGL((k_skinny_ring<NB, MT, D, DEQ>), dim3(grid), dim3((unsigned)(64 * nwave)), lds, s, qx, qw, sx,
                       sw, acc, y, M, N, K);
    return launch_status();
}

template <int NBA, int NBB, int MT, int D, bool DEQ>
static int32_t launch_ring_mixed(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc,
                                 float *y, int M, int N, int K, int cus, hipStream_t s)
{
    constexpr int nwave = 4;
    constexpr size_t lds = (size_t)nwave * D * (NBA + 2 * MT) * 1024;   // also covers the partial sums (<= 16 KB)
    static_assert(2 * lds <= 160 * 1024 && NBB == NBA - 1 && NBB >= 1, "two workgroups share a compute unit");
    if (N != 8 * cus * (NBA + NBB)) return MI_EINVAL;
    MI_LDS_OPT_IN((&k_skinny_ring_mixed<NBA, NBB, MT, D, DEQ>), 160 * 1024);
    hipLaunchKernelGGL((k_skinny_ring_mixed<NBA, NBB, MT, D, DEQ>), dim3((unsigned)(2 * cus)), dim3(64 * nwave), lds, s,
                       qx, qw, sx, sw, acc, y, M, N, K);
    return launch_status();
}

template <bool DEQ>
int32_t launch_skinny(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc,
                      float *y, int64_t M64, int64_t N64, int64_t K64, hipStream_t s)
{
    const int M = (int)M64, N = (int)N64, K = (int)K64;
    // M = 2..4 on a long K: the register kernel reads M activation rows per weight row pair and its activation
    // traffic passes the weight traffic; the ring kernel reads them once per 16 weight rows (measured 13.4 against
    // 16.6 us for 14336 -> 4096 at M = 4, a tie or worse on K = 4096)
    const bool reg_path = M == 1 || (M <= 4 && K < 8192);
    if (reg_path) {
        // K = 1024 * CW * QW (last chunk may be ragged) with CW <= 7 chunks per wave and QW in {1, 2, 4} waves per row
        const int nchunk = (K + 1023) >> 10;
        for (int QW = 1; QW <= 4; QW <<= 1) {
            if (nchunk % QW || nchunk / QW > 7) continue;
            const int CW = nchunk / QW;
            if (M == 1) return launch_reg_cw<1, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, CW, QW, s);
            if (M == 2) return launch_reg_cw<2, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, CW, QW, s);
            return launch_reg_cw<4, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, CW, QW, s);
        }
    }
    if (reg_path && (int64_t)4 * K <= 152 * 1024) {
        if (M == 1) return launch_dot4<1, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, s);
        if (M == 2) return launch_dot4<2, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, s);
        return launch_dot4<4, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, s);
    }
    const int cus = compute_units();
    const int steps = K >> 7;
    const int MT = (M + 15) / 16;
    // Up to 16 tokens and rows that deal out evenly: every compute unit gets the same number of 8-row blocks in two
    // workgroups of four waves (3, 5, 7 blocks a unit: one workgroup with a block more than the other; 10, 12, 14:
    // equal ones).  With 16-row workgroups on N = 6144 half of the units stream twice as many rows as the other half,
    // and on N = 14336 or 28672 a quarter of them four groups to the others' three.  Measured at M = 16, K = 4096,
    // weights from HBM: 9.17 -> 8.50 us (N = 6144), 14.8 -> 14.1 us (14336), 26.8 -> 24.4 us (28672).  N = 4096 stays
    // with one 16-row workgroup of eight waves per unit (two 8-row workgroups read the activation codes twice as
    // often: 17.2 against 14.4 us at K = 14336).
    if (MT == 1 && N % (8 * cus) == 0 && steps >= 8) {
        const int per_cu = N / (8 * cus);
        switch (per_cu) {
        case 3: return launch_ring_mixed<2, 1, 1, 4, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, cus, s);
        case 5: return launch_ring_mixed<3, 2, 1, 3, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, cus, s);
        case 7: return launch_ring_mixed<4, 3, 1, 3, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, cus, s);
        case 10: return launch_ring<5, 1, 2, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, 4, s);
        case 12: return launch_ring<6, 1, 2, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, 4, s);
        case 14: return launch_ring<7, 1, 2, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, 4, s);
        default: break;
        }
    }
    // Two 16-row groups per workgroup halve the activation traffic when there are rows enough to fill the
    // chip.  Four waves (a 64-72 KB ring set, so two workgroups share a compute unit and overlap their
    // prologues and epilogues) when there are workgroups enough, else eight waves to keep bytes in flight.
    const bool two = MT == 1 && N / 32 >= cus + cus / 2;
    const int wgs = two ? (N + 31) / 32 : (N + 15) / 16;
    int nwave = wgs >= cus + cus / 2 ? 4 : 8;
    while (nwave > 1 && nwave > steps) nwave >>= 1;
    switch (MT) {
    case 1:
        return two ? launch_ring<4, 1, 3, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, nwave, s)
                   : launch_ring<2, 1, 4, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, nwave, s);
    case 2: return launch_ring<2, 2, 2, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, nwave, s);
    case 3:
    case 4: return launch_ring<2, 4, 1, DEQ>(qx, sx, qw, sw, acc, y, M, N, K, nwave, s);
    default: return MI_ERANGE;
    }
}

template int32_t launch_skinny<true>(const int8_t *, const float *, const int8_t *, const float *, int32_t *,
                                     float *, int64_t, int64_t, int64_t, hipStream_t);
template int32_t launch_skinny<false>(const int8_t *, const float *, const int8_t *, const float *, int32_t *,
                                      float *, int64_t, int64_t, int64_t, hipStream_t);

}  // namespace mi
