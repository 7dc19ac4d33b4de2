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
// workgroup owns 16 gate + 16 up rows (or 64 down rows) of one expert, reads
// them from HBM once with 128-bit loads as MFMA A-fragments, and walks the
// expert's tokens 32 at a time with the gathered activation codes as B
// fragments.  Waves split K; partial accumulators meet in LDS.
//
// Bound: HBM on the int8 expert weights, E * 3 * H * I bytes per layer call.
#include "common.h"

namespace mi {
namespace moe {

constexpr int MAX_TOPK = 8;
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
template <int OFF, int N>
__device__ __forceinline__ void fold(float (&p)[64], int lane)
{
    const bool hi = (lane & OFF) != 0;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const float keep = hi ? p[i + N] : p[i];
        const float send = hi ? p[i] : p[i + N];
        p[i] = keep + shfl_xor_f(send, OFF);
    }
}

template <int MAX_THREADS>
__global__ __launch_bounds__(MAX_THREADS) void k_moe_route(const float *__restrict__ x,
                                                           const float *__restrict__ wr, int32_t *__restrict__ idx,
                                                           float *__restrict__ w, int T, int H, int E, int topk)
{
    __shared__ float s_logit[4][256];
    __shared__ float s_top[4][MAX_TOPK];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t0 = blockIdx.x * 4;
    const int e0 = wave * 16;

    float p[64];
#pragma unroll
    for (int i = 0; i < 64; ++i) p[i] = 0.0f;
    const float *xr[4];
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) xr[tt] = x + (int64_t)min(t0 + tt, T - 1) * H + 4 * lane;
    const float *wp = wr + (int64_t)e0 * H + 4 * lane;
    const int nj = e0 < E ? H / 256 : 0;  // waves past the last expert group only help with top-k
    for (int j = 0; j < nj; ++j) {
        float4 xv[4];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) xv[tt] = *reinterpret_cast<const float4 *>(xr[tt] + 256 * j);
        float4 wv[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) wv[e] = *reinterpret_cast<const float4 *>(wp + (int64_t)e * H + 256 * j);
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                float a = p[tt * 16 + e];
                a = __builtin_fmaf(xv[tt].x, wv[e].x, a);
                a = __builtin_fmaf(xv[tt].y, wv[e].y, a);
                a = __builtin_fmaf(xv[tt].z, wv[e].z, a);
                a = __builtin_fmaf(xv[tt].w, wv[e].w, a);
                p[tt * 16 + e] = a;
            }
    }
    fold<32, 32>(p, lane);
    fold<16, 16>(p, lane);
    fold<8, 8>(p, lane);
    fold<4, 4>(p, lane);
    fold<2, 2>(p, lane);
    fold<1, 1>(p, lane);
    // lane l now holds pair l: token l/16, expert e0 + l%16
    if (e0 < E) s_logit[lane >> 4][e0 + (lane & 15)] = p[0];
    __syncthreads();

    // top-k by rank counting: rank(i) = #{j : l_j > l_i or (l_j == l_i and j < i)}
    if (wave < 4 && t0 + wave < T) {
        const int t = t0 + wave;
        const float *lg = s_logit[wave];
        float mine[4];
        int rank[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = lane + 64 * u;
            mine[u] = i < E ? lg[i] : -INFINITY;
            rank[u] = 0;
        }
        for (int j = 0; j < E; ++j) {
            const float v = lg[j];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i = lane + 64 * u;
                rank[u] += (v > mine[u] || (v == mine[u] && j < i)) ? 1 : 0;
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = lane + 64 * u;
            if (i < E && rank[u] < topk) {
                idx[(int64_t)t * topk + rank[u]] = i;
                s_top[wave][rank[u]] = mine[u];
            }
        }
    }
    __syncthreads();
    if (wave < 4 && t0 + wave < T && lane < topk) {
        const float *tp = s_top[wave];
        float sum = 0.0f;
        for (int s = 0; s < topk; ++s) sum = sum + expf(tp[s] - tp[0]);
        w[(int64_t)(t0 + wave) * topk + lane] = expf(tp[lane] - tp[0]) / sum;
    }
}

// -------------------------------------------------------------- a10 dispatch
// One workgroup.  bm[e][t/32] bit t%32 = "token t picked expert e" (a token
// picks an expert at most once), so the stable rank of pair (t, slot) inside
// its expert is the number of set bits below t in row e.
__global__ __launch_bounds__(1024) void k_moe_dispatch(const int32_t *__restrict__ idx, int32_t *__restrict__ perm,
                                                       int32_t *__restrict__ seg_off, int T, int E, int topk)
{
    extern __shared__ uint32_t s_dyn[];
    const int W = (T + 31) >> 5;
    uint32_t *bm = s_dyn;                 // [E][W]
    uint32_t *pre = s_dyn + E * W;        // [E][W] exclusive popcount prefix
    int *seg = reinterpret_cast<int *>(s_dyn + 2 * E * W);  // [E+1]
    const int tid = threadIdx.x, nt = blockDim.x;
    const int P = T * topk;
    for (int i = tid; i < E * W; i += nt) bm[i] = 0u;
    __syncthreads();
    for (int pr = tid; pr < P; pr += nt) {
        const int e = idx[pr], t = pr / topk;
        if (e >= 0 && e < E) atomicOr(&bm[e * W + (t >> 5)], 1u << (t & 31));
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
    if (tid == 0) {
        seg[0] = 0;
        for (int e = 0; e < E; ++e) seg[e + 1] += seg[e];
    }
    __syncthreads();
    for (int e = tid; e <= E; e += nt) seg_off[e] = seg[e];
    for (int pr = tid; pr < P; pr += nt) {
        const int e = idx[pr], t = pr / topk;
        if (e < 0 || e >= E) continue;
        const uint32_t word = bm[e * W + (t >> 5)];
        const int pos = seg[e] + (int)pre[e * W + (t >> 5)] + __popc(word & ((1u << (t & 31)) - 1u));
        perm[pos] = pr;
    }
}

// ------------------------------------------------------- a11 grouped GEMMs
// Shared shape: a workgroup of 4 waves owns NG groups of 16 weight rows of one
// expert; wave w owns K steps [steps*w/4, steps*(w+1)/4).  Tokens of the expert
// are walked 32 at a time (two MFMA B-fragments).
constexpr int MT = 2;  // 16-token fragments per pass

// gate/up + SwiGLU.  Weight rows: 16 of wg and the same 16 of wu (NG = 2).
__global__ __launch_bounds__(256) void k_moe_gate_up(const int8_t *__restrict__ qx, const float *__restrict__ sx,
                                                     const int32_t *__restrict__ perm,
                                                     const int32_t *__restrict__ seg_off,
                                                     const int8_t *__restrict__ wg, const float *__restrict__ sg,
                                                     const int8_t *__restrict__ wu, const float *__restrict__ su,
                                                     float *__restrict__ h, int H, int I, int topk)
{
    __shared__ int s_part[4][2][MT][4][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int e = blockIdx.y, n0 = blockIdx.x * 16;
    const int seg0 = seg_off[e], count = seg_off[e + 1] - seg0;
    if (count <= 0) return;
    const int steps = H >> 6;
    const int s0 = steps * wave / 4, s1 = steps * (wave + 1) / 4;
    const int8_t *gp = wg + ((int64_t)e * I + n0 + r) * H + g * 16;
    const int8_t *up = wu + ((int64_t)e * I + n0 + r) * H + g * 16;

    for (int base = 0; base < count; base += 16 * MT) {
        const int8_t *xp[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int row = min(base + mt * 16 + r, count - 1);
            const int tok = perm[seg0 + row] / topk;
            xp[mt] = qx + (int64_t)tok * H + g * 16;
        }
        v4i ag[MT], au[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) { ag[mt] = (v4i){0, 0, 0, 0}; au[mt] = (v4i){0, 0, 0, 0}; }
#pragma unroll 4
        for (int s = s0; s < s1; ++s) {
            const v4i a_g = *reinterpret_cast<const v4i *>(gp + (int64_t)s * 64);
            const v4i a_u = *reinterpret_cast<const v4i *>(up + (int64_t)s * 64);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const v4i b = *reinterpret_cast<const v4i *>(xp[mt] + (int64_t)s * 64);
                ag[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_g, b, ag[mt], 0, 0, 0);
                au[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_u, b, au[mt], 0, 0, 0);
            }
        }
        __syncthreads();  // previous pass has finished reading s_part
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                s_part[wave][0][mt][c][lane] = ag[mt][c];
                s_part[wave][1][mt][c][lane] = au[mt][c];
            }
        __syncthreads();
        // 32 tokens x 16 channels: thread -> (token row, channel), channel fastest
        for (int o = tid; o < 16 * MT * 16; o += 256) {
            const int nl = o & 15, row = o >> 4;
            if (base + row >= count) continue;
            const int mt = row >> 4, src = (nl >> 2) * 16 + (row & 15), c = nl & 3;
            int sg_i = 0, su_i = 0;
#pragma unroll
            for (int wv = 0; wv < 4; ++wv) { sg_i += s_part[wv][0][mt][c][src]; su_i += s_part[wv][1][mt][c][src]; }
            const int pos = seg0 + base + row;
            const int tok = perm[pos] / topk;
            const float sxt = sx[tok];
            const float gv = ((float)sg_i * sxt) * sg[(int64_t)e * I + n0 + nl];
            const float uv = ((float)su_i * sxt) * su[(int64_t)e * I + n0 + nl];
            h[(int64_t)pos * I + n0 + nl] = (gv / (1.0f + expf(-gv))) * uv;
        }
    }
}

// down projection.  NG = 4 groups of 16 rows of wd per workgroup.
constexpr int NGD = 4;
__global__ __launch_bounds__(256) void k_moe_down(const int8_t *__restrict__ hq, const float *__restrict__ hs,
                                                  const int32_t *__restrict__ perm,
                                                  const int32_t *__restrict__ seg_off,
                                                  const int8_t *__restrict__ wd, const float *__restrict__ sd,
                                                  float *__restrict__ out, int H, int I)
{
    __shared__ int s_part[4][NGD][MT][4][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int e = blockIdx.y, n0 = blockIdx.x * 16 * NGD;
    const int seg0 = seg_off[e], count = seg_off[e + 1] - seg0;
    if (count <= 0) return;
    const int steps = I >> 6;
    const int s0 = steps * wave / 4, s1 = steps * (wave + 1) / 4;
    const int8_t *wp[NGD];
#pragma unroll
    for (int ng = 0; ng < NGD; ++ng) wp[ng] = wd + ((int64_t)e * H + min(n0 + ng * 16 + r, H - 1)) * I + g * 16;

    for (int base = 0; base < count; base += 16 * MT) {
        const int8_t *xp[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) xp[mt] = hq + (int64_t)(seg0 + min(base + mt * 16 + r, count - 1)) * I + g * 16;
        v4i acc[NGD][MT];
#pragma unroll
        for (int ng = 0; ng < NGD; ++ng)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[ng][mt] = (v4i){0, 0, 0, 0};
#pragma unroll 3
        for (int s = s0; s < s1; ++s) {
            v4i b[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) b[mt] = *reinterpret_cast<const v4i *>(xp[mt] + (int64_t)s * 64);
#pragma unroll
            for (int ng = 0; ng < NGD; ++ng) {
                const v4i a = *reinterpret_cast<const v4i *>(wp[ng] + (int64_t)s * 64);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[ng][mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b[mt], acc[ng][mt], 0, 0, 0);
            }
        }
        __syncthreads();
#pragma unroll
        for (int ng = 0; ng < NGD; ++ng)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int c = 0; c < 4; ++c) s_part[wave][ng][mt][c][lane] = acc[ng][mt][c];
        __syncthreads();
        for (int o = tid; o < 16 * MT * 16 * NGD; o += 256) {
            const int nl = o & (16 * NGD - 1), row = o / (16 * NGD);
            if (base + row >= count || n0 + nl >= H) continue;
            const int ng = nl >> 4, nn = nl & 15;
            const int mt = row >> 4, src = (nn >> 2) * 16 + (row & 15), c = nn & 3;
            int sum = 0;
#pragma unroll
            for (int wv = 0; wv < 4; ++wv) sum += s_part[wv][ng][mt][c][src];
            const int pos = seg0 + base + row;
            const int pair = perm[pos];
            out[(int64_t)pair * H + n0 + nl] = ((float)sum * hs[pos]) * sd[(int64_t)e * H + n0 + nl];
        }
    }
}

// y[t, n] = sum over slots in order of w[t, slot] * out[t*topk + slot, n]
__global__ __launch_bounds__(256) void k_moe_combine(const float *__restrict__ out, const float *__restrict__ w,
                                                     float *__restrict__ y, int T, int H, int topk)
{
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= (int64_t)T * H) return;
    const int t = (int)(i / H), n = (int)(i - (int64_t)t * H);
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s = 0; s < topk; ++s) {
        const float ws = w[(int64_t)t * topk + s];
        const float4 v = *reinterpret_cast<const float4 *>(out + ((int64_t)t * topk + s) * H + n);
        a.x = a.x + ws * v.x; a.y = a.y + ws * v.y; a.z = a.z + ws * v.z; a.w = a.w + ws * v.w;
    }
    *reinterpret_cast<float4 *>(y + i) = a;
}

static int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

struct Layout {
    int64_t off[10];
    int64_t total;
};

static Layout layout(int64_t T, int64_t H, int64_t I, int64_t E, int64_t topk)
{
    const int64_t P = T * topk;
    const int64_t sz[10] = {T * H, T * 4, P * 4, (E + 1) * 4, P * I * 4, P * I, P * 4, P * H * 4, P * 4, P * 4};
    Layout L;
    int64_t o = 0;
    for (int i = 0; i < 10; ++i) { L.off[i] = o; o += align_up(sz[i], 256); }
    L.total = o;
    return L;
}

static int32_t check_shapes(int64_t T, int64_t H, int64_t I, int64_t E, int32_t topk)
{
    if (T <= 0 || H <= 0 || I <= 0 || E <= 0 || topk <= 0) return MI_EINVAL;
    if (H % 128 || I % 256 || topk > MAX_TOPK || topk > E) return MI_EINVAL;
    if (H > 32768 || I > 32768 || T * topk > (1LL << 24) || E > 65535) return MI_ERANGE;
    if (2 * E * ((T + 31) / 32) + E + 1 > DISPATCH_MAX_WORDS) return MI_ERANGE;  // dispatch bitmap in LDS
    return MI_OK;
}

}  // namespace moe
}  // namespace mi

using namespace mi;

extern "C" int32_t mi_moe_route(const float *x, const float *wr, int32_t *idx, float *w, int64_t T, int64_t H,
                                int64_t E, int32_t topk, void *stream)
{
    if (!x || !wr || !idx || !w || T < 0 || H <= 0 || E <= 0 || topk <= 0) return MI_EINVAL;
    if (H % 256 || E % 16 || topk > moe::MAX_TOPK || topk > E) return MI_EINVAL;
    if (E > 256 || T > (1LL << 24)) return MI_ERANGE;
    if (!aligned16(x) || !aligned16(wr) || !aligned4(idx) || !aligned4(w)) return MI_EINVAL;
    if (T == 0) return MI_OK;
    const int waves = (int)(E / 16) < 4 ? 4 : (int)(E / 16);  // the top-k phase uses waves 0..3
    const dim3 grid((unsigned)((T + 3) / 4)), blk((unsigned)(64 * waves));
    if (waves <= 8)   // up to 128 experts: 512 threads, so a lane may keep 256 registers
        hipLaunchKernelGGL(moe::k_moe_route<512>, grid, blk, 0, as_stream(stream), x, wr, idx, w, (int)T, (int)H,
                           (int)E, (int)topk);
    else
        hipLaunchKernelGGL(moe::k_moe_route<1024>, grid, blk, 0, as_stream(stream), x, wr, idx, w, (int)T, (int)H,
                           (int)E, (int)topk);
    return launch_status();
}

extern "C" int32_t mi_moe_dispatch(const int32_t *idx, int32_t *perm, int32_t *seg_off, int64_t T, int64_t E,
                                   int32_t topk, void *stream)
{
    if (!idx || !perm || !seg_off || T < 0 || E <= 0 || topk <= 0) return MI_EINVAL;
    if (T * topk > (1LL << 24) || E > 65535) return MI_ERANGE;
    const int64_t words = 2 * E * ((T + 31) / 32) + E + 1;
    if (words > moe::DISPATCH_MAX_WORDS) return MI_ERANGE;
    static bool attr_set = false;  // idempotent; a race only repeats the call
    if (!attr_set) {
        MI_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&moe::k_moe_dispatch),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)(moe::DISPATCH_MAX_WORDS * 4)));
        attr_set = true;
    }
    hipLaunchKernelGGL(moe::k_moe_dispatch, dim3(1), dim3(1024), (size_t)words * 4, as_stream(stream), idx, perm,
                       seg_off, (int)T, (int)E, (int)topk);
    return launch_status();
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
    if (which < 0 || which > 9) return MI_EINVAL;
    return moe::layout(T, H, I, E, topk).off[which];
}

extern "C" int32_t mi_moe_ffn(const float *x, const int32_t *idx, const float *w, const int8_t *wg, const float *sg,
                              const int8_t *wu, const float *su, const int8_t *wd, const float *sd, float *y,
                              int64_t T, int64_t H, int64_t I, int64_t E, int32_t topk, void *workspace,
                              int64_t workspace_bytes, void *stream)
{
    int32_t rc = moe::check_shapes(T, H, I, E, topk);
    if (rc) return rc;
    if (!x || !idx || !w || !wg || !sg || !wu || !su || !wd || !sd || !y || !workspace) return MI_EINVAL;
    if (!aligned16(x) || !aligned16(wg) || !aligned16(wu) || !aligned16(wd) || !aligned16(y) || !aligned16(workspace))
        return MI_EINVAL;
    const moe::Layout L = moe::layout(T, H, I, E, topk);
    if (workspace_bytes < L.total) return MI_ENOSPC;
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

    rc = mi_moe_dispatch(idx, perm, seg, T, E, topk, stream);
    if (rc) return rc;
    rc = mi_fwht_quant_f32_i8(x, qx, sx, T, H, 128, stream);
    if (rc) return rc;
    hipLaunchKernelGGL(moe::k_moe_gate_up, dim3((unsigned)(I / 16), (unsigned)E), dim3(256), 0, s, qx, sx, perm, seg,
                       wg, sg, wu, su, h, (int)H, (int)I, (int)topk);
    rc = launch_status();
    if (rc) return rc;
    rc = mi_fwht_quant_f32_i8(h, hq, hs, P, I, 256, stream);
    if (rc) return rc;
    hipLaunchKernelGGL(moe::k_moe_down, dim3((unsigned)((H + 16 * moe::NGD - 1) / (16 * moe::NGD)), (unsigned)E),
                       dim3(256), 0, s, hq, hs, perm, seg, wd, sd, out, (int)H, (int)I);
    rc = launch_status();
    if (rc) return rc;
    hipLaunchKernelGGL(moe::k_moe_combine, dim3((unsigned)((T * H / 4 + 255) / 256)), dim3(256), 0, s, out, w, y,
                       (int)T, (int)H, (int)topk);
    return launch_status();
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
    char *ws = static_cast<char *>(workspace);
    int32_t *idx = reinterpret_cast<int32_t *>(ws + L.off[8]);
    float *w = reinterpret_cast<float *>(ws + L.off[9]);
    rc = mi_moe_route(x, wr, idx, w, T, H, E, topk, stream);
    if (rc) return rc;
    return mi_moe_ffn(x, idx, w, wg, sg, wu, su, wd, sd, y, T, H, I, E, topk, workspace, workspace_bytes, stream);
}
