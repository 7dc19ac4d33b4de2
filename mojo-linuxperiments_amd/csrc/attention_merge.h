// Merge of the partial results of a split decode attention, shared by the merge kernels (attention.hip) and by the
// split kernel that merges its own row when it is the last of the row's workgroups to finish (attention_tiled.hip).
#pragma once
#include "common.h"

namespace mi {
namespace attn {

// COHERENT: the values were written by other workgroups of the SAME kernel: they are read with agent-scope atomic
// loads, which do not hit in the compute unit's vector L1 (a line of the workspace may sit there from an earlier
// kernel or an earlier row of this one).
template <bool COHERENT>
__device__ __forceinline__ float ld1(const float *p)
{
    if constexpr (COHERENT) {
        return __builtin_bit_cast(float, __hip_atomic_load(reinterpret_cast<const unsigned *>(p), __ATOMIC_RELAXED,
                                                           __HIP_MEMORY_SCOPE_AGENT));
    } else {
        return *p;
    }
}
template <bool COHERENT>
__device__ __forceinline__ float4 ld4(const float *p)   // 16-byte aligned
{
    if constexpr (COHERENT) {
        const unsigned long long *q = reinterpret_cast<const unsigned long long *>(p);
        const unsigned long long a = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long b = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return make_float4(__uint_as_float((unsigned)a), __uint_as_float((unsigned)(a >> 32)),
                           __uint_as_float((unsigned)b), __uint_as_float((unsigned)(b >> 32)));
    } else {
        return *reinterpret_cast<const float4 *>(p);
    }
}

// Merge of the splits of one (b, h) row by the 16 lanes that own it (lane j: elements 4j..4j+3 and 64+4j..).
// SP > 0: the split count is known at compile time and every load of the row goes out before the first use (one
// memory round trip).  Returns the normalized row in the rotated basis of V.
template <int SP, bool COHERENT>
__device__ __forceinline__ void merge_row(const float *part_o, const float *part_ml,
                                          int splits_rt, int64_t bkv, int hl, int j, float (&v)[8])
{
    const int splits = SP > 0 ? SP : splits_rt;
    const float *ml0 = part_ml + bkv * splits * 8;
    const float *po0 = part_o + (bkv * splits * 4 + hl) * 128;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = 0.0f;
    float l = 0.0f;
    if constexpr (SP > 0) {
        float ms[SP], ls[SP];
        float4 lo[SP], hi[SP];
#pragma unroll
        for (int s = 0; s < SP; ++s) {
            ms[s] = ld1<COHERENT>(ml0 + s * 8 + hl);
            ls[s] = ld1<COHERENT>(ml0 + s * 8 + 4 + hl);
            lo[s] = ld4<COHERENT>(po0 + s * 4 * 128 + 4 * j);
            hi[s] = ld4<COHERENT>(po0 + s * 4 * 128 + 64 + 4 * j);
        }
        float mx = ms[0];
#pragma unroll
        for (int s = 1; s < SP; ++s) mx = fmaxf(mx, ms[s]);
#pragma unroll
        for (int s = 0; s < SP; ++s) {
            const float w = (ms[s] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(ms[s] - mx);   // empty split
            l = __builtin_fmaf(ls[s], w, l);
            v[0] = __builtin_fmaf(lo[s].x, w, v[0]); v[1] = __builtin_fmaf(lo[s].y, w, v[1]);
            v[2] = __builtin_fmaf(lo[s].z, w, v[2]); v[3] = __builtin_fmaf(lo[s].w, w, v[3]);
            v[4] = __builtin_fmaf(hi[s].x, w, v[4]); v[5] = __builtin_fmaf(hi[s].y, w, v[5]);
            v[6] = __builtin_fmaf(hi[s].z, w, v[6]); v[7] = __builtin_fmaf(hi[s].w, w, v[7]);
        }
    } else if (splits <= 8) {
        // a count known only at run time, but small: every load of the row still goes out before the first use (one
        // memory round trip); slots past the count repeat the last split and get weight 0
        float ms[8], ls[8];
        float4 lo[8], hi[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int s = min(i, splits - 1);
            ms[i] = ld1<COHERENT>(ml0 + s * 8 + hl);
            ls[i] = ld1<COHERENT>(ml0 + s * 8 + 4 + hl);
            lo[i] = ld4<COHERENT>(po0 + s * 4 * 128 + 4 * j);
            hi[i] = ld4<COHERENT>(po0 + s * 4 * 128 + 64 + 4 * j);
        }
        float mx = ms[0];
#pragma unroll
        for (int i = 1; i < 8; ++i) mx = fmaxf(mx, ms[i]);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float w = (i >= splits || ms[i] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(ms[i] - mx);
            l = __builtin_fmaf(ls[i], w, l);
            v[0] = __builtin_fmaf(lo[i].x, w, v[0]); v[1] = __builtin_fmaf(lo[i].y, w, v[1]);
            v[2] = __builtin_fmaf(lo[i].z, w, v[2]); v[3] = __builtin_fmaf(lo[i].w, w, v[3]);
            v[4] = __builtin_fmaf(hi[i].x, w, v[4]); v[5] = __builtin_fmaf(hi[i].y, w, v[5]);
            v[6] = __builtin_fmaf(hi[i].z, w, v[6]); v[7] = __builtin_fmaf(hi[i].w, w, v[7]);
        }
    } else {
        // any split count: the maxima first (one round trip), then the partials in batches of eight whose loads all
        // go out before the first use
        float mx = -INFINITY;
        for (int s0 = 0; s0 < splits; s0 += 8) {
            float ms[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) ms[i] = ld1<COHERENT>(ml0 + min(s0 + i, splits - 1) * 8 + hl);
#pragma unroll
            for (int i = 0; i < 8; ++i) mx = fmaxf(mx, ms[i]);
        }
        for (int s0 = 0; s0 < splits; s0 += 8) {
            float ms[8], ls[8];
            float4 lo[8], hi[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int s = min(s0 + i, splits - 1);
                ms[i] = ld1<COHERENT>(ml0 + s * 8 + hl);
                ls[i] = ld1<COHERENT>(ml0 + s * 8 + 4 + hl);
                lo[i] = ld4<COHERENT>(po0 + s * 4 * 128 + 4 * j);
                hi[i] = ld4<COHERENT>(po0 + s * 4 * 128 + 64 + 4 * j);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float w = (s0 + i >= splits || ms[i] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(ms[i] - mx);
                l = __builtin_fmaf(ls[i], w, l);
                v[0] = __builtin_fmaf(lo[i].x, w, v[0]); v[1] = __builtin_fmaf(lo[i].y, w, v[1]);
                v[2] = __builtin_fmaf(lo[i].z, w, v[2]); v[3] = __builtin_fmaf(lo[i].w, w, v[3]);
                v[4] = __builtin_fmaf(hi[i].x, w, v[4]); v[5] = __builtin_fmaf(hi[i].y, w, v[5]);
                v[6] = __builtin_fmaf(hi[i].z, w, v[6]); v[7] = __builtin_fmaf(hi[i].w, w, v[7]);
            }
        }
    }
    const float rl = l > 0.0f ? 1.0f / l : 0.0f;   // a sequence of length 0 gives a row of zeros
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] *= rl;
}

}  // namespace attn
}  // namespace mi
