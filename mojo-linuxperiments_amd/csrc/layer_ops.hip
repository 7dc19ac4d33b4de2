// The small fp32 operators that sit between the int8 kernels in one decoder layer of a decode step:
// residual add + RMSNorm, rotary embedding fused with the KV-cache append, SwiGLU on a fused gate|up row.
// None of them exists upstream (the upstream repository holds no model code); they follow the CPU oracle's
// decisions D10-D12.  All are bound by launch latency at decode sizes (a few hundred KB per call).
#include "fwht_core.h"

namespace mi {
namespace layer {

// y[m,:] = (h * r) * g with h = x (+ res), r = 1 / sqrt(mean(h^2) + eps); h is also written when res is given.
// One workgroup per row, C float4 per thread (H <= 4096 * C).
template <int C>
__global__ __launch_bounds__(256) void k_add_rmsnorm(const float *__restrict__ x, const float *__restrict__ res,
                                                     const float *__restrict__ g, float eps,
                                                     float *__restrict__ h_out, float *__restrict__ y, int H)
{
    __shared__ float s_part[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t row = (int64_t)blockIdx.x * H;
    float4 v[C];
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < C; ++i) {
        const int col = 4 * (tid + 256 * i);
        if (col < H) {
            v[i] = *reinterpret_cast<const float4 *>(x + row + col);
            if (res) {
                const float4 r4 = *reinterpret_cast<const float4 *>(res + row + col);
                v[i].x = v[i].x + r4.x; v[i].y = v[i].y + r4.y; v[i].z = v[i].z + r4.z; v[i].w = v[i].w + r4.w;
                *reinterpret_cast<float4 *>(h_out + row + col) = v[i];
            }
            ss += v[i].x * v[i].x;
            ss += v[i].y * v[i].y;
            ss += v[i].z * v[i].z;
            ss += v[i].w * v[i].w;
        } else {
            v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) ss += __shfl_xor(ss, off, 64);
    if (lane == 0) s_part[wave] = ss;
    __syncthreads();
    const float total = (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
    const float r = 1.0f / sqrtf(total / (float)H + eps);
#pragma unroll
    for (int i = 0; i < C; ++i) {
        const int col = 4 * (tid + 256 * i);
        if (col < H) {
            const float4 g4 = *reinterpret_cast<const float4 *>(g + col);
            float4 o;
            o.x = (v[i].x * r) * g4.x; o.y = (v[i].y * r) * g4.y; o.z = (v[i].z * r) * g4.z; o.w = (v[i].w * r) * g4.w;
            *reinterpret_cast<float4 *>(y + row + col) = o;
        }
    }
}

// One decode token per sequence, rows of [Hq query heads | Hkv key heads | Hkv value heads] x 128 floats: query
// and key heads get the rotary embedding of the sequence's position (pairs (i, i + 64), angles from the caller's
// cos / sin tables [T_cap, 64]); queries leave packed as [B, Hq, 128]; keys and values are rotated (block Hadamard
// 128) and quantized like any cache row and stored at that position of the cache.  16 lanes per head.
__global__ __launch_bounds__(256) void k_rope_kv_append(const float *__restrict__ qkv, int64_t row_stride,
                                                        const float *__restrict__ cs, const float *__restrict__ sn,
                                                        float *__restrict__ q_out, int8_t *__restrict__ kq, float *__restrict__ ks,
                                                        int8_t *__restrict__ vq, float *__restrict__ vs,
                                                        const int32_t *__restrict__ pos, int B, int Hq, int Hkv,
                                                        int T_cap)
{
    constexpr int D = 128, LPB = 16;
    const int t = threadIdx.x, j = t % LPB;
    const int heads = Hq + 2 * Hkv;
    const int flat = blockIdx.x * 16 + t / LPB;
    const int b = min(flat / heads, B - 1), hd = flat % heads;
    const int tp = pos[b];
    const bool live = flat < B * heads && tp >= 0 && tp < T_cap;
    const float *src = qkv + (int64_t)b * row_stride + (int64_t)hd * D + 4 * j;
    float v[8];
    if (live) {
        const float4 lo = *reinterpret_cast<const float4 *>(src);
        const float4 hi = *reinterpret_cast<const float4 *>(src + D / 2);
        v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w;
        v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = 0.0f;
    }
    const bool is_q = hd < Hq, is_v = hd >= Hq + Hkv;
    if (live && !is_v) {
        const float4 c4 = *reinterpret_cast<const float4 *>(cs + (int64_t)tp * (D / 2) + 4 * j);
        const float4 s4 = *reinterpret_cast<const float4 *>(sn + (int64_t)tp * (D / 2) + 4 * j);
        const float c[4] = {c4.x, c4.y, c4.z, c4.w}, s[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float a = v[e], bb = v[e + 4];
            v[e] = a * c[e] - bb * s[e];
            v[e + 4] = bb * c[e] + a * s[e];
        }
        if (is_q) {
            float *dst = q_out + ((int64_t)b * Hq + hd) * D + 4 * j;
            *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
            *reinterpret_cast<float4 *>(dst + D / 2) = make_float4(v[4], v[5], v[6], v[7]);
        }
    }
    // every lane takes part in the cross-lane stages; query heads simply do not store
    fwht_chunk<D>(v, j);
    float a = abs8(v);
#pragma unroll
    for (int m = LPB / 2; m >= 1; m >>= 1) a = fmaxf(a, __shfl_xor(a, m, 64));
    const float sc = (a == 0.0f) ? 1.0f : a / 127.0f;
    const float inv = (a == 0.0f) ? 0.0f : 127.0f / a;
    if (live && !is_q) {
        const int h = is_v ? hd - Hq - Hkv : hd - Hq;
        const int64_t row = ((int64_t)b * Hkv + h) * T_cap + tp;
        int8_t *q = (is_v ? vq : kq) + row * D + 4 * j;
        if (j == 0) (is_v ? vs : ks)[row] = sc;
        *reinterpret_cast<uint32_t *>(q) = quant4(v[0], v[1], v[2], v[3], inv);
        *reinterpret_cast<uint32_t *>(q + D / 2) = quant4(v[4], v[5], v[6], v[7], inv);
    }
}

// h[m, n] = silu(gu[m, n]) * gu[m, I + n]: gate and up come out of one projection as one row of 2*I
__global__ __launch_bounds__(256) void k_swiglu(const float *__restrict__ gu, float *__restrict__ h, int64_t M, int I)
{
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= M * I) return;
    const int64_t m = i / I;
    const int n = (int)(i - m * I);
    const float4 g = *reinterpret_cast<const float4 *>(gu + m * 2 * I + n);
    const float4 u = *reinterpret_cast<const float4 *>(gu + m * 2 * I + I + n);
    float4 o;
    o.x = (g.x / (1.0f + expf(-g.x))) * u.x;
    o.y = (g.y / (1.0f + expf(-g.y))) * u.y;
    o.z = (g.z / (1.0f + expf(-g.z))) * u.z;
    o.w = (g.w / (1.0f + expf(-g.w))) * u.w;
    *reinterpret_cast<float4 *>(h + i) = o;
}

// The row operators fused with the rotate + quantize prologue of the linear that follows them, so that a decode
// step launches one kernel where it launched two and the normalized / activated row never travels as fp32 unless
// the caller asks for it.  One workgroup per row, thread t owns chunks t, t + TPB, ... (C of them) in the layout
// of fwht_core.h; the arithmetic per element is that of the separate kernels in the same order.
// MODE 0: v = ((x (+ res)) * r) * g (RMSNorm);  MODE 1: v = silu(gate) * up from a fused [gate | up] row.
template <int BLOCK, int C, int MODE, int TPB>
__global__ __launch_bounds__(TPB) void k_row_op_quant(const float *__restrict__ x, const float *__restrict__ res,
                                                      const float *__restrict__ g, float eps,
                                                      float *__restrict__ h_out, float *__restrict__ y_out,
                                                      int8_t *__restrict__ q, float *__restrict__ scale, int K)
{
    constexpr int LPB = BLOCK / 8;
    constexpr int NW = TPB / 64;
    __shared__ float s_part[C * NW], s_max[NW];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int j = t % LPB;
    const int nchunk = K / 8;
    const int64_t row = blockIdx.x;
    float v[C][8];
    int base[C];
    float ss[C];   // sums of squares per chunk, then per group of 64 chunks (group wave + i * NW)
#pragma unroll
    for (int i = 0; i < C; ++i) {
        ss[i] = 0.0f;
        const int c = t + i * TPB;
        base[i] = (c / LPB) * BLOCK + 4 * j;
        if (c < nchunk) {
            if constexpr (MODE == 0) {
                const float *xr = x + row * (int64_t)K + base[i];
                float4 lo = *reinterpret_cast<const float4 *>(xr), hi = *reinterpret_cast<const float4 *>(xr + BLOCK / 2);
                if (res) {
                    const float *rr = res + row * (int64_t)K + base[i];
                    const float4 rl = *reinterpret_cast<const float4 *>(rr), rh = *reinterpret_cast<const float4 *>(rr + BLOCK / 2);
                    lo.x = lo.x + rl.x; lo.y = lo.y + rl.y; lo.z = lo.z + rl.z; lo.w = lo.w + rl.w;
                    hi.x = hi.x + rh.x; hi.y = hi.y + rh.y; hi.z = hi.z + rh.z; hi.w = hi.w + rh.w;
                    float *ho = h_out + row * (int64_t)K + base[i];
                    *reinterpret_cast<float4 *>(ho) = lo;
                    *reinterpret_cast<float4 *>(ho + BLOCK / 2) = hi;
                }
                v[i][0] = lo.x; v[i][1] = lo.y; v[i][2] = lo.z; v[i][3] = lo.w;
                v[i][4] = hi.x; v[i][5] = hi.y; v[i][6] = hi.z; v[i][7] = hi.w;
                ss[i] = chunk_sumsq(v[i]);
            } else {
                const float *gr = x + row * 2 * (int64_t)K + base[i];
                const float4 gl = *reinterpret_cast<const float4 *>(gr), gh = *reinterpret_cast<const float4 *>(gr + BLOCK / 2);
                const float4 ul = *reinterpret_cast<const float4 *>(gr + K), uh = *reinterpret_cast<const float4 *>(gr + K + BLOCK / 2);
                const float gg[8] = {gl.x, gl.y, gl.z, gl.w, gh.x, gh.y, gh.z, gh.w};
                const float uu[8] = {ul.x, ul.y, ul.z, ul.w, uh.x, uh.y, uh.z, uh.w};
#pragma unroll
                for (int e = 0; e < 8; ++e) v[i][e] = (gg[e] / (1.0f + expf(-gg[e]))) * uu[e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[i][e] = 0.0f;
        }
    }
    if constexpr (MODE == 0) {
        // the norm weights are requested before the reduction: their round trip runs under it
        float4 gl[C], gh[C];
#pragma unroll
        for (int i = 0; i < C; ++i) {
            if (t + i * TPB < nchunk) {
                gl[i] = *reinterpret_cast<const float4 *>(g + base[i]);
                gh[i] = *reinterpret_cast<const float4 *>(g + base[i] + BLOCK / 2);
            }
        }
#pragma unroll
        for (int i = 0; i < C; ++i) {
            ss[i] = group_sum(ss[i]);
            if (lane == 0) s_part[wave + i * NW] = ss[i];
        }
        __syncthreads();
        const float total = tree_sum<C * NW>(s_part);   // the order of fwht_core.h: the same bits whatever TPB is
        const float r = 1.0f / sqrtf(total / (float)K + eps);
#pragma unroll
        for (int i = 0; i < C; ++i) {
            if (t + i * TPB < nchunk) {
                v[i][0] = (v[i][0] * r) * gl[i].x; v[i][1] = (v[i][1] * r) * gl[i].y;
                v[i][2] = (v[i][2] * r) * gl[i].z; v[i][3] = (v[i][3] * r) * gl[i].w;
                v[i][4] = (v[i][4] * r) * gh[i].x; v[i][5] = (v[i][5] * r) * gh[i].y;
                v[i][6] = (v[i][6] * r) * gh[i].z; v[i][7] = (v[i][7] * r) * gh[i].w;
            }
        }
    }
    if (y_out) {
        float *yo = y_out + row * (int64_t)K;
#pragma unroll
        for (int i = 0; i < C; ++i) {
            if (t + i * TPB < nchunk) {
                *reinterpret_cast<float4 *>(yo + base[i]) = make_float4(v[i][0], v[i][1], v[i][2], v[i][3]);
                *reinterpret_cast<float4 *>(yo + base[i] + BLOCK / 2) = make_float4(v[i][4], v[i][5], v[i][6], v[i][7]);
            }
        }
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < C; ++i) {
        fwht_chunk<BLOCK>(v[i], j);
        amax = fmaxf(amax, abs8(v[i]));
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if (lane == 0) s_max[wave] = amax;
    __syncthreads();
    float a = s_max[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) a = fmaxf(a, s_max[w]);
    const float sc = (a == 0.0f) ? 1.0f : a / 127.0f;
    const float inv = (a == 0.0f) ? 0.0f : 127.0f / a;
    if (t == 0) scale[row] = sc;
    int8_t *qrow = q + row * (int64_t)K;
#pragma unroll
    for (int i = 0; i < C; ++i) {
        if (t + i * TPB < nchunk) {
            *reinterpret_cast<uint32_t *>(qrow + base[i]) = quant4(v[i][0], v[i][1], v[i][2], v[i][3], inv);
            *reinterpret_cast<uint32_t *>(qrow + base[i] + BLOCK / 2) = quant4(v[i][4], v[i][5], v[i][6], v[i][7], inv);
        }
    }
}

template <int BLOCK, int MODE>
static int32_t launch_row_op_quant(const float *x, const float *res, const float *g, float eps, float *h_out,
                                   float *y_out, int8_t *q, float *scale, int64_t M, int64_t K, hipStream_t s)
{
    // few rows (a decode step): a row is worth a whole compute unit, 1024 threads hold at most two chunks each
    const int64_t nchunk = K / 8;
    const dim3 grid((unsigned)M);
#define MI_ROWQ(CC, TT)                                                                                           \
    hipLaunchKernelGGL((k_row_op_quant<BLOCK, CC, MODE, TT>), grid, dim3(TT), 0, s, x, res, g, eps, h_out, y_out, q, \
                       scale, (int)K)
    if (nchunk <= 256) MI_ROWQ(1, 256);
    else if (nchunk <= 512) MI_ROWQ(1, 512);
    else if (nchunk <= 1024) MI_ROWQ(1, 1024);
    else if (nchunk <= 2048) MI_ROWQ(2, 1024);
    else return MI_ERANGE;
#undef MI_ROWQ
    return launch_status();
}

__global__ __launch_bounds__(256) void k_add(const float *__restrict__ a, const float *__restrict__ b,
                                             float *__restrict__ out, int64_t n)
{
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n) return;
    const float4 x = *reinterpret_cast<const float4 *>(a + i), y = *reinterpret_cast<const float4 *>(b + i);
    *reinterpret_cast<float4 *>(out + i) = make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w);
}

}  // namespace layer
}  // namespace mi

using namespace mi;

extern "C" int32_t mi_rmsnorm_f32(const float *x, const float *residual, const float *g, float eps, float *h_out,
                                  float *y, int64_t M, int64_t H, void *stream)
{
    if (!x || !g || !y || M < 0 || H <= 0 || !(eps >= 0.0f)) return MI_EINVAL;
    if (residual && !h_out) return MI_EINVAL;
    if (H % 4) return MI_EINVAL;
    if (H > 16384 || M > 0x7fffffffLL) return MI_ERANGE;
    if (!aligned16(x) || !aligned16(g) || !aligned16(y) || (residual && (!aligned16(residual) || !aligned16(h_out))))
        return MI_EINVAL;
    if (M == 0) return MI_OK;
    const int C = (int)((H / 4 + 255) / 256);
    const dim3 grid((unsigned)M);
#define MI_NORM(CC)                                                                                              \
    hipLaunchKernelGGL(layer::k_add_rmsnorm<CC>, grid, dim3(256), 0, as_stream(stream), x, residual, g, eps, h_out, \
                       y, (int)H)
    if (C <= 1) MI_NORM(1);
    else if (C <= 2) MI_NORM(2);
    else if (C <= 4) MI_NORM(4);
    else if (C <= 8) MI_NORM(8);
    else MI_NORM(16);
#undef MI_NORM
    return launch_status();
}

extern "C" int32_t mi_rope_kv_append_f32_i8(const float *qkv, int64_t row_stride, const float *rope_cos,
                                            const float *rope_sin, float *q_out, int8_t *kq, float *ks, int8_t *vq,
                                            float *vs,
                                            const int32_t *pos, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                                            int64_t T_cap, void *stream)
{
    if (!qkv || !rope_cos || !rope_sin || !q_out || !kq || !ks || !vq || !vs || !pos) return MI_EINVAL;
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || T_cap <= 0 || D != 128) return MI_EINVAL;
    if (row_stride < (Hq + 2 * Hkv) * D || row_stride % 4) return MI_EINVAL;
    if (B * (Hq + 2 * Hkv) > (1LL << 24) || T_cap > (1LL << 24)) return MI_ERANGE;
    if (!aligned16(qkv) || !aligned16(rope_cos) || !aligned16(rope_sin) || !aligned16(q_out) || !aligned4(kq) || !aligned4(vq) ||
        !aligned4(ks) || !aligned4(vs) || !aligned4(pos))
        return MI_EINVAL;
    const int64_t rows = B * (Hq + 2 * Hkv);
    hipLaunchKernelGGL(layer::k_rope_kv_append, dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, as_stream(stream),
                       qkv, row_stride, rope_cos, rope_sin, q_out, kq, ks, vq, vs, pos, (int)B, (int)Hq, (int)Hkv,
                       (int)T_cap);
    return launch_status();
}

extern "C" int32_t mi_swiglu_f32(const float *gate_up, float *h, int64_t M, int64_t I, void *stream)
{
    if (!gate_up || !h || M < 0 || I <= 0 || I % 4) return MI_EINVAL;
    if (M * I > (1LL << 40)) return MI_ERANGE;
    if (!aligned16(gate_up) || !aligned16(h)) return MI_EINVAL;
    if (M == 0) return MI_OK;
    const int64_t quads = M * I / 4;
    hipLaunchKernelGGL(layer::k_swiglu, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, as_stream(stream),
                       gate_up, h, M, (int)I);
    return launch_status();
}

extern "C" int32_t mi_rmsnorm_quant_f32_i8(const float *x, const float *residual, const float *g, float eps,
                                           float *h_out, float *y_out, int8_t *q, float *scale, int64_t M,
                                           int64_t H, int32_t block, void *stream)
{
    if (!x || !g || !q || !scale || M < 0 || H <= 0 || !(eps >= 0.0f)) return MI_EINVAL;
    if (residual && !h_out) return MI_EINVAL;
    if ((block != 128 && block != 256) || H % block) return MI_EINVAL;
    if (H > 16384 || M > 0x7fffffffLL) return MI_ERANGE;
    if (!aligned16(x) || !aligned16(g) || !aligned4(q) || !aligned4(scale) || (y_out && !aligned16(y_out)) ||
        (residual && (!aligned16(residual) || !aligned16(h_out))))
        return MI_EINVAL;
    if (M == 0) return MI_OK;
    return block == 128 ? layer::launch_row_op_quant<128, 0>(x, residual, g, eps, h_out, y_out, q, scale, M, H, as_stream(stream))
                        : layer::launch_row_op_quant<256, 0>(x, residual, g, eps, h_out, y_out, q, scale, M, H, as_stream(stream));
}

extern "C" int32_t mi_swiglu_quant_f32_i8(const float *gate_up, float *h_out, int8_t *q, float *scale, int64_t M,
                                          int64_t I, int32_t block, void *stream)
{
    if (!gate_up || !q || !scale || M < 0 || I <= 0) return MI_EINVAL;
    if ((block != 128 && block != 256) || I % block) return MI_EINVAL;
    if (I > 16384 || M > 0x7fffffffLL) return MI_ERANGE;
    if (!aligned16(gate_up) || !aligned4(q) || !aligned4(scale) || (h_out && !aligned16(h_out))) return MI_EINVAL;
    if (M == 0) return MI_OK;
    return block == 128 ? layer::launch_row_op_quant<128, 1>(gate_up, nullptr, nullptr, 0.0f, nullptr, h_out, q, scale, M, I, as_stream(stream))
                        : layer::launch_row_op_quant<256, 1>(gate_up, nullptr, nullptr, 0.0f, nullptr, h_out, q, scale, M, I, as_stream(stream));
}

extern "C" int32_t mi_add_f32(const float *a, const float *b, float *out, int64_t n, void *stream)
{
    if (!a || !b || !out || n < 0 || n % 4) return MI_EINVAL;
    if (!aligned16(a) || !aligned16(b) || !aligned16(out)) return MI_EINVAL;
    if (n == 0) return MI_OK;
    hipLaunchKernelGGL(layer::k_add, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, as_stream(stream), a, b,
                       out, n);
    return launch_status();
}
