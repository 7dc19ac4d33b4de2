// Block Hadamard rotation fused with the symmetric int8 row quantizer
// (workload elements a1 + a2, reused for weight prep a3 and KV-cache rows a7).
//
// Data layout.  A row of K floats is cut into chunks of 8 floats; chunk c of a
// Hadamard block of size BLOCK is the two float4 at offsets 4c and
// BLOCK/2 + 4c inside the block, so one thread owns the elements whose index
// bits are {0,1} (inside a float4) and the top bit (lower / upper half), and
// the BLOCK/8 consecutive lanes that share a block own the middle bits.  The
// butterfly stages therefore run in the fixed order h = 1, 2 (in-lane),
// h = 4 .. BLOCK/4 (lane xor 1, 2, 4, 8[, 16] through DPP / ds_swizzle),
// h = BLOCK/2 (in-lane), each output being one fp32 add or subtract, followed
// by one multiply by fp32(1/sqrt(BLOCK)).  That is the order the CPU
// restatement uses, and since no FMA is formed (-ffp-contract=off) the codes
// are bit-exact against it.
//
// Every load is a float4 and the BLOCK/8 neighbouring lanes of a block read
// 2*BLOCK contiguous bytes (whole 128-byte lines); the codes leave as one
// dword per float4.  The kernel reads 4 B and writes 1 B per element: HBM-bound.
#include "common.h"
#include "fwht_core.h"

namespace mi {

// One workgroup per row; thread t owns chunks t, t + T, ... (C of them).
// QUANT: write int8 codes + scale; otherwise write the rotated fp32 row.
template <int BLOCK, int C, bool QUANT>
__device__ __forceinline__ void fwht_row_body(const float *x, int8_t *__restrict__ q, float *__restrict__ scale,
                                              float *xrot, int K, int64_t row)
{
    constexpr int LPB = BLOCK / 8;
    const int t = threadIdx.x, T = blockDim.x;
    const int j = t % LPB;
    const int nchunk = K / 8;
    const float *xr = x + row * (int64_t)K;

    float v[C][8];
    int base[C];
#pragma unroll
    for (int i = 0; i < C; ++i) {
        const int c = t + i * T;
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
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < C; ++i) {
        fwht_chunk<BLOCK>(v[i], j);
        amax = fmaxf(amax, abs8(v[i]));
    }

    if constexpr (!QUANT) {
        float *orow = xrot + row * (int64_t)K;
#pragma unroll
        for (int i = 0; i < C; ++i) {
            if (t + i * T < nchunk) {
                *reinterpret_cast<float4 *>(orow + base[i]) = make_float4(v[i][0], v[i][1], v[i][2], v[i][3]);
                *reinterpret_cast<float4 *>(orow + base[i] + BLOCK / 2) = make_float4(v[i][4], v[i][5], v[i][6], v[i][7]);
            }
        }
    } else {
        // row absmax: wave butterfly, then across waves through LDS
        __shared__ float s_max[16];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
        const int wave = t >> 6, nwave = (T + 63) >> 6;
        if ((t & 63) == 0) s_max[wave] = amax;
        __syncthreads();
        float a = s_max[0];
        for (int w = 1; w < nwave; ++w) a = fmaxf(a, s_max[w]);
        const float sc = (a == 0.0f) ? 1.0f : a / 127.0f;
        const float inv = (a == 0.0f) ? 0.0f : 127.0f / a;
        if (t == 0) scale[row] = sc;
        int8_t *qrow = q + row * (int64_t)K;
#pragma unroll
        for (int i = 0; i < C; ++i) {
            if (t + i * T < nchunk) {
                *reinterpret_cast<uint32_t *>(qrow + base[i]) = quant4(v[i][0], v[i][1], v[i][2], v[i][3], inv);
                *reinterpret_cast<uint32_t *>(qrow + base[i] + BLOCK / 2) = quant4(v[i][4], v[i][5], v[i][6], v[i][7], inv);
            }
        }
    }
}

template <int BLOCK, int C, bool QUANT>
__global__ __launch_bounds__(256) void k_fwht_rows(const float *x, int8_t *__restrict__ q,
                                                    float *__restrict__ scale, float *xrot, int K)
{
    fwht_row_body<BLOCK, C, QUANT>(x, q, scale, xrot, K, (int64_t)blockIdx.x);
}

// Several row sets in ONE launch (the prefill step's three rotate + quantize prologues): workgroup b finds its set
// by the sets' cumulative row counts and runs the body of k_fwht_rows on its row, with the chunk count of that set's
// K.  Same code per row, hence the same codes and scales as separate launches; 256 threads, K >= 2048.
constexpr int QUANT_BATCH_MAX = 8;
struct QuantSet {
    const float *x;
    int8_t *q;
    float *scale;
    int K;
    int first_row;   // of this set in the grid
};
struct QuantBatch {
    QuantSet s[QUANT_BATCH_MAX];
    int n;
};
// CMAX: the most 8-float chunks per thread any set of the batch needs.  The kernel's registers are those of its
// widest row body whichever set a workgroup works on, so a batch of rows up to K = 14336 is not made to run at the
// occupancy of the K = 32768 body (160 registers, three waves per SIMD).
template <int BLOCK, int CMAX>
__global__ __launch_bounds__(256) void k_fwht_rows_batch(const QuantBatch b)
{
    int i = 0;
#pragma unroll
    for (int k = 1; k < QUANT_BATCH_MAX; ++k)
        if (k < b.n && (int)blockIdx.x >= b.s[k].first_row) i = k;
    const QuantSet &S = b.s[i];
    const int64_t row = (int64_t)blockIdx.x - S.first_row;
    const int C = (S.K / 8 + 255) / 256;
    if (C <= 1) fwht_row_body<BLOCK, 1, true>(S.x, S.q, S.scale, nullptr, S.K, row);
    else if (C <= 2) fwht_row_body<BLOCK, 2, true>(S.x, S.q, S.scale, nullptr, S.K, row);
    else if constexpr (CMAX <= 2) return;
    else if (C <= 4) fwht_row_body<BLOCK, 4, true>(S.x, S.q, S.scale, nullptr, S.K, row);
    else if constexpr (CMAX <= 4) return;
    else if (C <= 7) fwht_row_body<BLOCK, 7, true>(S.x, S.q, S.scale, nullptr, S.K, row);
    else if constexpr (CMAX <= 7) return;
    else if (C <= 8) fwht_row_body<BLOCK, 8, true>(S.x, S.q, S.scale, nullptr, S.K, row);
    else fwht_row_body<BLOCK, 16, true>(S.x, S.q, S.scale, nullptr, S.K, row);
}

// Short rows (K <= 2048): one wave per row, four rows per workgroup; lane l owns chunks l, l + 64, ...
// The absmax never leaves the wave, so there is no LDS and no barrier.
template <int BLOCK, int C, bool QUANT>
__global__ __launch_bounds__(256) void k_fwht_wave(const float *x, int8_t *__restrict__ q, float *__restrict__ scale,
                                                   float *xrot, int K, int64_t M)
{
    constexpr int LPB = BLOCK / 8;
    const int lane = threadIdx.x & 63;
    const int j = lane % LPB;
    const int nchunk = K / 8;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;
    const float *xr = x + row * (int64_t)K;
    float v[C][8];
    int base[C];
#pragma unroll
    for (int i = 0; i < C; ++i) {
        const int c = lane + i * 64;
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
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < C; ++i) {
        fwht_chunk<BLOCK>(v[i], j);
        amax = fmaxf(amax, abs8(v[i]));
    }
    if constexpr (!QUANT) {
        float *orow = xrot + row * (int64_t)K;
#pragma unroll
        for (int i = 0; i < C; ++i) {
            if (lane + i * 64 < nchunk) {
                *reinterpret_cast<float4 *>(orow + base[i]) = make_float4(v[i][0], v[i][1], v[i][2], v[i][3]);
                *reinterpret_cast<float4 *>(orow + base[i] + BLOCK / 2) = make_float4(v[i][4], v[i][5], v[i][6], v[i][7]);
            }
        }
    } else {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
        const float sc = (amax == 0.0f) ? 1.0f : amax / 127.0f;
        const float inv = (amax == 0.0f) ? 0.0f : 127.0f / amax;
        if (lane == 0) scale[row] = sc;
        int8_t *qrow = q + row * (int64_t)K;
#pragma unroll
        for (int i = 0; i < C; ++i) {
            if (lane + i * 64 < nchunk) {
                *reinterpret_cast<uint32_t *>(qrow + base[i]) = quant4(v[i][0], v[i][1], v[i][2], v[i][3], inv);
                *reinterpret_cast<uint32_t *>(qrow + base[i] + BLOCK / 2) = quant4(v[i][4], v[i][5], v[i][6], v[i][7], inv);
            }
        }
    }
}

// K == BLOCK (a row is one Hadamard block, e.g. attention heads and KV-cache
// rows): BLOCK/8 lanes per row, 256*8/BLOCK rows per workgroup, the absmax is
// reduced inside the lane group only.
template <int BLOCK, bool QUANT>
__global__ __launch_bounds__(256) void k_fwht_small(const float *x, int8_t *__restrict__ q,
                                                    float *__restrict__ scale, float *xrot, int64_t M)
{
    constexpr int LPB = BLOCK / 8;
    constexpr int ROWS = 256 / LPB;
    const int t = threadIdx.x, j = t % LPB;
    const int64_t row = (int64_t)blockIdx.x * ROWS + t / LPB;
    const bool live = row < M;
    const int64_t off = row * BLOCK + 4 * j;
    float v[8];
    if (live) {
        const float4 lo = *reinterpret_cast<const float4 *>(x + off);
        const float4 hi = *reinterpret_cast<const float4 *>(x + off + BLOCK / 2);
        v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w;
        v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = 0.0f;
    }
    fwht_chunk<BLOCK>(v, j);
    if constexpr (!QUANT) {
        if (live) {
            *reinterpret_cast<float4 *>(xrot + off) = make_float4(v[0], v[1], v[2], v[3]);
            *reinterpret_cast<float4 *>(xrot + off + BLOCK / 2) = make_float4(v[4], v[5], v[6], v[7]);
        }
    } else {
        float a = abs8(v);
#pragma unroll
        for (int m = LPB / 2; m >= 1; m >>= 1) a = fmaxf(a, __shfl_xor(a, m, 64));
        const float sc = (a == 0.0f) ? 1.0f : a / 127.0f;
        const float inv = (a == 0.0f) ? 0.0f : 127.0f / a;
        if (live) {
            if (j == 0) scale[row] = sc;
            *reinterpret_cast<uint32_t *>(q + off) = quant4(v[0], v[1], v[2], v[3], inv);
            *reinterpret_cast<uint32_t *>(q + off + BLOCK / 2) = quant4(v[4], v[5], v[6], v[7], inv);
        }
    }
}

// KV-cache append: the new token's key and value heads (128 floats each) are rotated and quantized exactly as
// k_fwht_small<128> does, and the codes and the scale land at position pos[b] of sequence b in the cache
// [B, Hkv, T_cap, 128] / [B, Hkv, T_cap].  16 lanes per head, 16 heads per workgroup; blockIdx.y = 0: keys, 1: values.
__global__ __launch_bounds__(256) void k_kv_append(const float *__restrict__ k_new, const float *__restrict__ v_new,
                                                   int64_t row_stride, int8_t *__restrict__ kq,
                                                   float *__restrict__ ks, int8_t *__restrict__ vq,
                                                   float *__restrict__ vs, const int32_t *__restrict__ pos, int B,
                                                   int Hkv, int T_cap, const int32_t *__restrict__ block_table,
                                                   int max_pages, int page_shift)
{
    constexpr int BLOCK = 128, LPB = 16;
    const int t = threadIdx.x, j = t % LPB;
    const int head = blockIdx.x * 16 + t / LPB;      // flat (b, h)
    const bool is_v = blockIdx.y != 0;
    const int b = min(head / Hkv, B - 1), h = head % Hkv;
    const int tp = pos[b];
    const bool live = head < B * Hkv && tp >= 0 && tp < T_cap;
    const float *src = (is_v ? v_new : k_new) + (int64_t)b * row_stride + (int64_t)h * BLOCK + 4 * j;
    float v[8];
    if (live) {
        const float4 lo = *reinterpret_cast<const float4 *>(src);
        const float4 hi = *reinterpret_cast<const float4 *>(src + BLOCK / 2);
        v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w;
        v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = 0.0f;
    }
    fwht_chunk<BLOCK>(v, j);
    float a = abs8(v);
#pragma unroll
    for (int m = LPB / 2; m >= 1; m >>= 1) a = fmaxf(a, __shfl_xor(a, m, 64));
    const float sc = (a == 0.0f) ? 1.0f : a / 127.0f;
    const float inv = (a == 0.0f) ? 0.0f : 127.0f / a;
    if (live) {
        int64_t row = ((int64_t)b * Hkv + h) * T_cap + tp;
        if (block_table) {
            // paged pool [page][kv head][P tokens]: the page that holds token tp of sequence b
            const int page = block_table[(int64_t)b * max_pages + (tp >> page_shift)];
            row = (((int64_t)page * Hkv + h) << page_shift) + (tp & ((1 << page_shift) - 1));
        }
        int8_t *q = (is_v ? vq : kq) + row * BLOCK + 4 * j;
        if (j == 0) (is_v ? vs : ks)[row] = sc;
        *reinterpret_cast<uint32_t *>(q) = quant4(v[0], v[1], v[2], v[3], inv);
        *reinterpret_cast<uint32_t *>(q + BLOCK / 2) = quant4(v[4], v[5], v[6], v[7], inv);
    }
}

template <int BLOCK, bool QUANT>
static int32_t launch_rows(const float *x, int8_t *q, float *scale, float *xrot, int64_t M, int64_t K,
                           hipStream_t s)
{
    if (K == BLOCK) {
        constexpr int ROWS = 256 / (BLOCK / 8);
        const int64_t grid = (M + ROWS - 1) / ROWS;
        hipLaunchKernelGGL((k_fwht_small<BLOCK, QUANT>), dim3((unsigned)grid), dim3(256), 0, s, x, q, scale, xrot, M);
        return launch_status();
    }
    const int nchunk = (int)(K / 8);
    if (nchunk <= 256 && M >= 1024) {
        // many short rows: a wave per row
        const dim3 grid((unsigned)((M + 3) / 4));
        const int CW = (nchunk + 63) / 64;
#define MI_WAVE_CASE(CC)                                                                                    \
    hipLaunchKernelGGL((k_fwht_wave<BLOCK, CC, QUANT>), grid, dim3(256), 0, s, x, q, scale, xrot, (int)K, M)
        if (CW <= 1) MI_WAVE_CASE(1);
        else if (CW <= 2) MI_WAVE_CASE(2);
        else MI_WAVE_CASE(4);
#undef MI_WAVE_CASE
        return launch_status();
    }
    int T = nchunk >= 256 ? 256 : ((nchunk + 63) / 64) * 64;
    const int C = (nchunk + T - 1) / T;
    const dim3 grid((unsigned)M), blk((unsigned)T);
#define MI_ROWS_CASE(CC)                                                                                   \
    hipLaunchKernelGGL((k_fwht_rows<BLOCK, CC, QUANT>), grid, blk, 0, s, x, q, scale, xrot, (int)K)
    if (C <= 1) MI_ROWS_CASE(1);
    else if (C <= 2) MI_ROWS_CASE(2);
    else if (C <= 4) MI_ROWS_CASE(4);
    else if (C <= 7) MI_ROWS_CASE(7);
    else if (C <= 8) MI_ROWS_CASE(8);
    else if (C <= 16) MI_ROWS_CASE(16);
    else return MI_ERANGE;
#undef MI_ROWS_CASE
    return launch_status();
}

static int32_t check_rows(const void *x, const void *out, int64_t M, int64_t K, int32_t block)
{
    if (!x || !out || M < 0 || K <= 0) return MI_EINVAL;
    if (block != 128 && block != 256) return MI_EINVAL;
    if (K % block) return MI_EINVAL;
    if (K > 32768 || M > 0x7fffffffLL) return MI_ERANGE;
    if (!aligned16(x)) return MI_EINVAL;
    return MI_OK;
}

}  // namespace mi

using namespace mi;

extern "C" int32_t mi_fwht_quant_f32_i8(const float *x, int8_t *q, float *scale, int64_t M, int64_t K,
                                        int32_t block, void *stream)
{
    int32_t rc = check_rows(x, q, M, K, block);
    if (rc) return rc;
    if (!scale || !aligned4(q) || !aligned4(scale)) return MI_EINVAL;
    if (M == 0) return MI_OK;
    return block == 128 ? launch_rows<128, true>(x, q, scale, nullptr, M, K, as_stream(stream))
                        : launch_rows<256, true>(x, q, scale, nullptr, M, K, as_stream(stream));
}

extern "C" int32_t mi_fwht_quant_batch_f32_i8(const mi_quant_rows *sets, int32_t n, int32_t block, void *stream)
{
    if (!sets || n < 1 || n > QUANT_BATCH_MAX) return MI_EINVAL;
    QuantBatch b = {};
    int64_t rows = 0;
    bool one_launch = true;
    for (int i = 0; i < n; ++i) {
        const mi_quant_rows &s = sets[i];
        int32_t rc = check_rows(s.x, s.q, s.M, s.K, block);
        if (rc) return rc;
        if (!s.scale || !aligned4(s.q) || !aligned4(s.scale)) return MI_EINVAL;
        // the batched kernel is the row-per-workgroup form at 256 threads; shorter rows (or a set without rows)
        // take the single launches, whose results are the same
        if (s.K < 2048 || s.M == 0) one_launch = false;
        b.s[i].x = s.x;
        b.s[i].q = s.q;
        b.s[i].scale = s.scale;
        b.s[i].K = (int)s.K;
        b.s[i].first_row = (int)rows;
        rows += s.M;
    }
    if (rows > 0x7fffffffLL) return MI_ERANGE;
    if (!one_launch) {
        for (int i = 0; i < n; ++i) {
            int32_t rc = mi_fwht_quant_f32_i8(sets[i].x, sets[i].q, sets[i].scale, sets[i].M, sets[i].K, block, stream);
            if (rc) return rc;
        }
        return MI_OK;
    }
    b.n = n;
    int cmax = 1;
    for (int i = 0; i < n; ++i) cmax = std::max(cmax, (b.s[i].K / 8 + 255) / 256);
#define MI_QBATCH(BLOCK_, CMAX_) \
    hipLaunchKernelGGL((k_fwht_rows_batch<BLOCK_, CMAX_>), dim3((unsigned)rows), dim3(256), 0, as_stream(stream), b)
    if (block == 128) {
        if (cmax <= 2) MI_QBATCH(128, 2);
        else if (cmax <= 4) MI_QBATCH(128, 4);
        else if (cmax <= 7) MI_QBATCH(128, 7);
        else MI_QBATCH(128, 16);
    } else {
        if (cmax <= 2) MI_QBATCH(256, 2);
        else if (cmax <= 4) MI_QBATCH(256, 4);
        else if (cmax <= 7) MI_QBATCH(256, 7);
        else MI_QBATCH(256, 16);
    }
#undef MI_QBATCH
    return launch_status();
}

extern "C" int32_t mi_kv_append_f32_i8(const float *k_new, const float *v_new, int64_t row_stride, int8_t *kq,
                                       float *ks, int8_t *vq, float *vs, const int32_t *pos, int64_t B,
                                       int64_t Hkv, int64_t D, int64_t T_cap, void *stream)
{
    if (!k_new || !v_new || !kq || !ks || !vq || !vs || !pos) return MI_EINVAL;
    if (B <= 0 || Hkv <= 0 || T_cap <= 0 || D != 128) return MI_EINVAL;
    if (row_stride < Hkv * D || row_stride % 4) return MI_EINVAL;
    if (B * Hkv > (1LL << 24) || T_cap > (1LL << 24)) return MI_ERANGE;
    if (!aligned16(k_new) || !aligned16(v_new) || !aligned4(kq) || !aligned4(vq) || !aligned4(ks) || !aligned4(vs) ||
        !aligned4(pos))
        return MI_EINVAL;
    const dim3 grid((unsigned)((B * Hkv + 15) / 16), 2);
    hipLaunchKernelGGL(k_kv_append, grid, dim3(256), 0, as_stream(stream), k_new, v_new, row_stride, kq, ks, vq, vs,
                       pos, (int)B, (int)Hkv, (int)T_cap, (const int32_t *)nullptr, 0, 0);
    return launch_status();
}

extern "C" int32_t mi_kv_append_paged_f32_i8(const float *k_new, const float *v_new, int64_t row_stride,
                                             int8_t *kq_pool, float *ks_pool, int8_t *vq_pool, float *vs_pool,
                                             const int32_t *block_table, int64_t max_pages, int64_t page_size,
                                             const int32_t *pos, int64_t B, int64_t Hkv, int64_t D, void *stream)
{
    if (!k_new || !v_new || !kq_pool || !ks_pool || !vq_pool || !vs_pool || !pos || !block_table) return MI_EINVAL;
    if (B <= 0 || Hkv <= 0 || D != 128 || max_pages <= 0) return MI_EINVAL;
    if (page_size < 16 || (page_size & (page_size - 1)) || page_size > (1 << 20)) return MI_EINVAL;
    if (row_stride < Hkv * D || row_stride % 4) return MI_EINVAL;
    if (B * Hkv > (1LL << 24) || max_pages * page_size > (1LL << 24)) return MI_ERANGE;
    if (!aligned16(k_new) || !aligned16(v_new) || !aligned4(kq_pool) || !aligned4(vq_pool) || !aligned4(ks_pool) ||
        !aligned4(vs_pool) || !aligned4(pos) || !aligned4(block_table))
        return MI_EINVAL;
    int shift = 0;
    while ((1LL << shift) < page_size) ++shift;
    const dim3 grid((unsigned)((B * Hkv + 15) / 16), 2);
    // positions are valid inside the sequence's table: [0, max_pages * page_size)
    hipLaunchKernelGGL(k_kv_append, grid, dim3(256), 0, as_stream(stream), k_new, v_new, row_stride, kq_pool, ks_pool,
                       vq_pool, vs_pool, pos, (int)B, (int)Hkv, (int)(max_pages * page_size), block_table,
                       (int)max_pages, shift);
    return launch_status();
}

extern "C" int32_t mi_fwht_f32(const float *x, float *out, int64_t M, int64_t K, int32_t block, void *stream)
{
    int32_t rc = check_rows(x, out, M, K, block);
    if (rc) return rc;
    if (!aligned16(out)) return MI_EINVAL;
    if (M == 0) return MI_OK;
    return block == 128 ? launch_rows<128, false>(x, nullptr, nullptr, out, M, K, as_stream(stream))
                        : launch_rows<256, false>(x, nullptr, nullptr, out, M, K, as_stream(stream));
}
