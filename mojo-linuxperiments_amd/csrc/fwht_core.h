// Device-side core of the block Hadamard rotation and the int8 row quantizer, shared by the stand-alone
// kernels and by the decode GEMV that quantizes its own activations.  A chunk is 8 floats of one Hadamard
// block (the two float4 at offsets 4j and BLOCK/2 + 4j, j = lane % (BLOCK/8)); the butterfly stages run in the
// fixed order h = 1, 2 (in-lane), 4 .. BLOCK/4 (across lanes), BLOCK/2 (in-lane), one fp32 add or subtract each.
#pragma once
#include "common.h"

namespace mi {

// value held by lane (lane ^ MASK); MASK in {1,2,4,8,16}
template <int MASK>
__device__ __forceinline__ float xor_lane(float v)
{
    const int i = __float_as_int(v);
    int r;
    if constexpr (MASK == 1) {
        r = __builtin_amdgcn_update_dpp(i, i, 0xB1, 0xf, 0xf, false);  // quad_perm [1,0,3,2]
    } else if constexpr (MASK == 2) {
        r = __builtin_amdgcn_update_dpp(i, i, 0x4E, 0xf, 0xf, false);  // quad_perm [2,3,0,1]
    } else {
        // ds_swizzle bit mode: lane' = ((lane & 0x1f) | 0) ^ MASK inside each half wave
        r = __builtin_amdgcn_ds_swizzle(i, 0x1F | (MASK << 10));
    }
    return __int_as_float(r);
}

// one cross-lane butterfly stage on 8 values: the lane whose MASK bit is
// clear holds x[i] and keeps x[i] + x[i+h]; its partner keeps x[i] - x[i+h]
template <int MASK>
__device__ __forceinline__ void cross_stage(float (&v)[8], unsigned negmask)
{
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float other = xor_lane<MASK>(v[e]);
        const float mine = __int_as_float(__float_as_int(v[e]) ^ negmask);  // -v on the upper lane
        v[e] = other + mine;
    }
}

template <int BLOCK>
__device__ __forceinline__ void fwht_chunk(float (&v)[8], int j)
{
    // h = 1, 2: inside each float4
#pragma unroll
    for (int b = 0; b < 8; b += 4) {
        float a0 = v[b] + v[b + 1], a1 = v[b] - v[b + 1];
        float a2 = v[b + 2] + v[b + 3], a3 = v[b + 2] - v[b + 3];
        v[b] = a0 + a2; v[b + 2] = a0 - a2;
        v[b + 1] = a1 + a3; v[b + 3] = a1 - a3;
    }
    // h = 4 .. BLOCK/4: across the lanes of the block
    cross_stage<1>(v, (j & 1) ? 0x80000000u : 0u);
    cross_stage<2>(v, (j & 2) ? 0x80000000u : 0u);
    cross_stage<4>(v, (j & 4) ? 0x80000000u : 0u);
    cross_stage<8>(v, (j & 8) ? 0x80000000u : 0u);
    if constexpr (BLOCK == 256) cross_stage<16>(v, (j & 16) ? 0x80000000u : 0u);
    // h = BLOCK/2: lower half against upper half
    constexpr float S = (BLOCK == 128) ? 0.08838834764831845f : 0.0625f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float lo = v[e] + v[e + 4], hi = v[e] - v[e + 4];
        v[e] = lo * S;
        v[e + 4] = hi * S;
    }
}

__device__ __forceinline__ float abs8(const float (&v)[8])
{
    float a = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) a = fmaxf(a, fabsf(v[e]));
    return a;
}

// Sum of squares of a row in an order that depends on the row alone and not on how many threads share it, so that
// a kernel of 256 threads and one of 1024 produce the same bits: the eight squares of a chunk are added in element
// order, the 64 chunks of a group (chunk index / 64, one wave's worth) by a xor butterfly (every lane ends with
// the same bits, a + b being b + a), and the groups pairwise in index order (tree_sum; absent groups count as 0,
// which changes nothing).
__device__ __forceinline__ float chunk_sumsq(const float (&v)[8])
{
    float s = v[0] * v[0];
#pragma unroll
    for (int e = 1; e < 8; ++e) s += v[e] * v[e];
    return s;
}
__device__ __forceinline__ float group_sum(float s)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
    return s;
}
template <int G>
__device__ __forceinline__ float tree_sum(const float *part)   // part[0 .. G-1], any G >= 1
{
    constexpr int P = G <= 1 ? 1 : 1 << (32 - __builtin_clz(G - 1));
    float t[P];
#pragma unroll
    for (int w = 0; w < P; ++w) t[w] = w < G ? part[w] : 0.0f;
#pragma unroll
    for (int n = P; n > 1; n >>= 1)
#pragma unroll
        for (int w = 0; w < n / 2; ++w) t[w] = t[2 * w] + t[2 * w + 1];
    return t[0];
}

__device__ __forceinline__ uint32_t quant4(float a, float b, float c, float d, float inv)
{
    const int i0 = (int)fminf(fmaxf(rintf(a * inv), -127.0f), 127.0f);
    const int i1 = (int)fminf(fmaxf(rintf(b * inv), -127.0f), 127.0f);
    const int i2 = (int)fminf(fmaxf(rintf(c * inv), -127.0f), 127.0f);
    const int i3 = (int)fminf(fmaxf(rintf(d * inv), -127.0f), 127.0f);
    return (uint32_t)(i0 & 0xff) | ((uint32_t)(i1 & 0xff) << 8) | ((uint32_t)(i2 & 0xff) << 16) |
           ((uint32_t)i3 << 24);
}

}  // namespace mi
