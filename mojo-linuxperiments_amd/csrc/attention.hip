// Grouped-query decode attention over an int8 KV cache (workload element a8).
//
//   per (b, h):  q' = quant(FWHT128(q))            int8 codes qq, scale sq
//                dot_t = qq . kq[b, h/G, t, :]      int32
//                s_t = dot_t * sq * ks_t / sqrt(D)
//                o' = sum_t softmax(s)_t * vs_t * vq[b, h/G, t, :]
//   and, unless the caller wants the rotated basis, o = FWHT128(o').
//
// Split-KV: grid = (splits, B*Hkv); a workgroup (4 waves) streams one span of
// tokens of one KV head once and serves the G = Hq/Hkv <= 4 query heads that
// share it.  A second small kernel merges the splits.
//
// Both passes load 16 bytes per lane in token-major order (lane l: token l/8
// of an 8-token group, bytes 16*(l%8)..+15), i.e. 1 KB contiguous per wave
// instruction, eight instructions in flight per wave.
// Pass 1 (scores).  Each lane runs v_dot4_i32_i8 of its 16 key bytes against
// the matching 16 query-code bytes of the G heads; the 8 lanes of a token add
// their int32 partial sums (lane xor 1, 2, 4).  Scores (already in log2 units)
// go to LDS, the running max stays in registers.
// Pass 2 (P.V).  v_mfma_f32_4x4x1_16B_f32 treats each aligned group of
// four lanes as one 4x4 outer product: the four lanes share a token, lane
// l%4 = i supplies p(token, head i) * vs(token) as the A value and one V
// element as the B value, so register i of the accumulator is head i.  Sixteen
// such MFMAs (one per byte of the lane's 16) consume a load; int8 -> fp32 is
// v_cvt_f32_ubyteN on (byte ^ 0x80) and the bias 128 * sum(p*vs) is removed
// once at the end.  The fp32 matrix pipe does the 4-head FMA work that would
// otherwise cost 64 VALU FMAs per 16 bytes.
//
// Bound: HBM.  Algorithmic bytes = K and V codes (2*B*Hkv*T*D) + their scales
// (8*B*Hkv*T) + q and o (8*B*Hq*D).
#include "common.h"

namespace mi {

namespace attn {

constexpr int D = 128;

template <int MASK>
__device__ __forceinline__ float lane_xor(float v)
{
    const int i = __float_as_int(v);
    int r;
    if constexpr (MASK == 1) r = __builtin_amdgcn_update_dpp(i, i, 0xB1, 0xf, 0xf, false);
    else if constexpr (MASK == 2) r = __builtin_amdgcn_update_dpp(i, i, 0x4E, 0xf, 0xf, false);
    else if constexpr (MASK < 32) r = __builtin_amdgcn_ds_swizzle(i, 0x1F | (MASK << 10));
    else r = __shfl_xor(i, 32, 64);
    return __int_as_float(r);
}

// normalized 128-point Hadamard over 16 lanes x 8 values, stage order h = 1, 2, ..., 64
__device__ __forceinline__ void fwht128(float (&v)[8], int j)
{
#pragma unroll
    for (int b = 0; b < 8; b += 4) {
        float a0 = v[b] + v[b + 1], a1 = v[b] - v[b + 1];
        float a2 = v[b + 2] + v[b + 3], a3 = v[b + 2] - v[b + 3];
        v[b] = a0 + a2; v[b + 2] = a0 - a2;
        v[b + 1] = a1 + a3; v[b + 3] = a1 - a3;
    }
#define MI_STAGE(MASK)                                                                              \
    {                                                                                               \
        const unsigned neg = (j & MASK) ? 0x80000000u : 0u;                                         \
        _Pragma("unroll") for (int e = 0; e < 8; ++e)                                               \
        {                                                                                           \
            const float other = lane_xor<MASK>(v[e]);                                               \
            v[e] = other + __int_as_float(__float_as_int(v[e]) ^ neg);                              \
        }                                                                                           \
    }
    MI_STAGE(1) MI_STAGE(2) MI_STAGE(4) MI_STAGE(8)
#undef MI_STAGE
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float lo = v[e] + v[e + 4], hi = v[e] - v[e + 4];
        v[e] = lo * 0.08838834764831845f;
        v[e + 4] = hi * 0.08838834764831845f;
    }
}

__device__ __forceinline__ uint32_t quant4(float a, float b, float c, float d, float inv)
{
    const int i0 = (int)fminf(fmaxf(rintf(a * inv), -127.0f), 127.0f);
    const int i1 = (int)fminf(fmaxf(rintf(b * inv), -127.0f), 127.0f);
    const int i2 = (int)fminf(fmaxf(rintf(c * inv), -127.0f), 127.0f);
    const int i3 = (int)fminf(fmaxf(rintf(d * inv), -127.0f), 127.0f);
    return (uint32_t)(i0 & 0xff) | ((uint32_t)(i1 & 0xff) << 8) | ((uint32_t)(i2 & 0xff) << 16) | ((uint32_t)i3 << 24);
}

struct Params {
    const float *q;
    const int8_t *kq;
    const float *ks;
    const int8_t *vq;
    const float *vs;
    float *part_o;   // [B*Hkv, splits, 4, 128]
    float *part_ml;  // [B*Hkv, splits, 2, 4]   (max in log2 units, sum)
    int8_t *dump_qq;
    float *dump_sq;
    int32_t *dump_dots;
    int Hq, Hkv, G, T;
    int tiles_per_split;  // 16-token tiles
    float score_scale;    // log2(e) / sqrt(D)
};

// value of lane (lane ^ OFF) for OFF in {8, 16, 32}
template <int OFF>
__device__ __forceinline__ float slot_xor(float v)
{
    const int i = __float_as_int(v);
    int r;
    if constexpr (OFF == 8) r = __builtin_amdgcn_update_dpp(0, i, 0x128, 0xf, 0xf, true);   // row_ror:8
    else if constexpr (OFF == 16) r = __builtin_amdgcn_ds_swizzle(i, 0x401F);
    else r = __shfl_xor(i, 32, 64);
    return __int_as_float(r);
}
// one round of the transposed butterfly over token slots: keep the half of the values whose index bit
// matches this lane's OFF bit, hand the other half to lane ^ OFF
template <int V, int OFF>
__device__ __forceinline__ void fold_slots(float (&p)[64], int lane)
{
    const bool hi = (lane & OFF) != 0;
#pragma unroll
    for (int i = 0; i < V / 2; ++i) {
        const float keep = hi ? p[i + V / 2] : p[i];
        const float send = hi ? p[i] : p[i + V / 2];
        p[i] = keep + slot_xor<OFF>(send);
    }
}

constexpr int WAVE_GROUPS = 16;   // 8-token groups per wave: a workgroup covers at most 4 * 16 * 8 = 512 tokens

template <bool DUMP>
__global__ __launch_bounds__(256) void k_gqa_split(Params p)
{
    __shared__ __attribute__((aligned(16))) int8_t s_q[4][4][D];
    __shared__ float s_sq[4][4];
    __shared__ float s_red[4][4][D];
    __shared__ float s_m[4][4], s_l[4][4], s_c[4][4];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int split = blockIdx.x, bkv = blockIdx.y;
    const int b = bkv / p.Hkv, kvh = bkv % p.Hkv;
    const int G = p.G, T = p.T;
    const int ntiles = (T + 15) >> 4;
    const int tile_lo = split * p.tiles_per_split;
    const int tile_hi = min(tile_lo + p.tiles_per_split, ntiles);
    // lane layout of both passes: token slot = l/8 of an 8-token group, 16-byte chunk = l%8; head = l%4
    const int hh = lane & 3, slot = lane >> 3, chunk = lane & 7;
    const int t_lo = tile_lo << 4;
    const int ngroups = max(0, min(tile_hi << 4, T) - t_lo + 7) >> 3;   // 8-token groups of this split
    const int8_t *kbase = p.kq + (int64_t)bkv * T * D + 16 * chunk;
    const int8_t *vbase = p.vq + (int64_t)bkv * T * D + 16 * chunk;
    const float *ksb = p.ks + (int64_t)bkv * T;
    const float *vsb = p.vs + (int64_t)bkv * T;

    // ---- every K byte of this wave and the first half of its V bytes are requested before anything else:
    // one load = 8 tokens x 128 B contiguous; wave w takes groups w, w+4, ...
    v4i kv[WAVE_GROUPS], va[WAVE_GROUPS / 2];
    float ksv[WAVE_GROUPS], vsa[WAVE_GROUPS / 2];
#pragma unroll
    for (int u = 0; u < WAVE_GROUPS; ++u) {
        const int tk = min(t_lo + (wave + 4 * u) * 8 + slot, T - 1);
        kv[u] = *reinterpret_cast<const v4i *>(kbase + (int64_t)tk * D);
        ksv[u] = ksb[tk];
    }
#pragma unroll
    for (int u = 0; u < WAVE_GROUPS / 2; ++u) {
        const int tk = min(t_lo + (wave + 4 * u) * 8 + slot, T - 1);
        va[u] = *reinterpret_cast<const v4i *>(vbase + (int64_t)tk * D);
        vsa[u] = vsb[tk];
    }

    // ---- query heads of this group: rotate, quantize, park the codes in LDS
    {
        const int hr = lane >> 4, jj = lane & 15;
        const int head = kvh * G + min(hr, G - 1);
        const float *qr = p.q + ((int64_t)b * p.Hq + head) * D;
        const float4 lo = *reinterpret_cast<const float4 *>(qr + 4 * jj);
        const float4 hi = *reinterpret_cast<const float4 *>(qr + 64 + 4 * jj);
        float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        fwht128(v, jj);
        float a = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) a = fmaxf(a, fabsf(v[e]));
        a = fmaxf(a, lane_xor<1>(a));
        a = fmaxf(a, lane_xor<2>(a));
        a = fmaxf(a, lane_xor<4>(a));
        a = fmaxf(a, lane_xor<8>(a));
        const float sc = (a == 0.0f) ? 1.0f : a / 127.0f;
        const float inv = (a == 0.0f) ? 0.0f : 127.0f / a;
        const uint32_t c0 = quant4(v[0], v[1], v[2], v[3], inv), c1 = quant4(v[4], v[5], v[6], v[7], inv);
        *reinterpret_cast<uint32_t *>(&s_q[wave][hr][4 * jj]) = c0;
        *reinterpret_cast<uint32_t *>(&s_q[wave][hr][64 + 4 * jj]) = c1;
        if (jj == 0) s_sq[wave][hr] = sc;
        if constexpr (DUMP) {
            if (split == 0 && wave == 0 && hr < G) {
                int8_t *dq = p.dump_qq + ((int64_t)b * p.Hq + head) * D;
                *reinterpret_cast<uint32_t *>(dq + 4 * jj) = c0;
                *reinterpret_cast<uint32_t *>(dq + 64 + 4 * jj) = c1;
                if (jj == 0) p.dump_sq[(int64_t)b * p.Hq + head] = sc;
            }
        }
    }
    __syncthreads();
    v4i qd[4];       // query codes of the 4 heads for this lane's chunk
#pragma unroll
    for (int h = 0; h < 4; ++h)
        qd[h] = h < G ? *reinterpret_cast<const v4i *>(&s_q[wave][h][16 * chunk]) : (v4i){0, 0, 0, 0};
    const float cq = hh < G ? s_sq[wave][hh] * p.score_scale : 0.0f;   // per-head factor of the score, log2 units

    // ---- pass 1: scores.  v_dot4_i32_i8 against the 4 heads, then the 8 lanes of a token add up
    // (xor 1, 2, 4).  The score of (token l/8, head l%4) stays in a register, in log2 units.
    float sc[WAVE_GROUPS];
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < WAVE_GROUPS; ++u) {
        const int gi = wave + 4 * u;
        const int tt = t_lo + gi * 8 + slot;
        int d[4];
#pragma unroll
        for (int h = 0; h < 4; ++h) {
            int a = __builtin_amdgcn_sdot4(kv[u][0], qd[h][0], 0, false);
            a = __builtin_amdgcn_sdot4(kv[u][1], qd[h][1], a, false);
            a = __builtin_amdgcn_sdot4(kv[u][2], qd[h][2], a, false);
            a = __builtin_amdgcn_sdot4(kv[u][3], qd[h][3], a, false);
            a += __builtin_amdgcn_update_dpp(0, a, 0xB1, 0xf, 0xf, true);   // lane ^ 1
            a += __builtin_amdgcn_update_dpp(0, a, 0x4E, 0xf, 0xf, true);   // lane ^ 2
            a += __builtin_amdgcn_ds_swizzle(a, 0x101F);                    // lane ^ 4
            d[h] = a;
        }
        const int mine = hh == 0 ? d[0] : hh == 1 ? d[1] : hh == 2 ? d[2] : d[3];
        const bool live = gi < ngroups && tt < T;
        sc[u] = live ? (float)mine * (ksv[u] * cq) : -INFINITY;
        if constexpr (DUMP) {
            if (live && hh < G && chunk < 4) p.dump_dots[((int64_t)b * p.Hq + kvh * G + hh) * T + tt] = mine;
        }
        mx = fmaxf(mx, sc[u]);
    }
    // the key registers are free: request the second half of V
    v4i vb[WAVE_GROUPS / 2];
    float vsb2[WAVE_GROUPS / 2];
#pragma unroll
    for (int u = 0; u < WAVE_GROUPS / 2; ++u) {
        const int tk = min(t_lo + (wave + 4 * (u + WAVE_GROUPS / 2)) * 8 + slot, T - 1);
        vb[u] = *reinterpret_cast<const v4i *>(vbase + (int64_t)tk * D);
        vsb2[u] = vsb[tk];
    }
    // lanes that share l%4 hold partial maxima of head l%4
    mx = fmaxf(mx, slot_xor<8>(mx));
    mx = fmaxf(mx, slot_xor<16>(mx));
    mx = fmaxf(mx, slot_xor<32>(mx));
    if (lane < 4) s_m[wave][lane] = mx;
    __syncthreads();

    // ---- pass 2: P.V on the fp32 matrix pipe
    const float m_h = fmaxf(fmaxf(s_m[0][hh], s_m[1][hh]), fmaxf(s_m[2][hh], s_m[3][hh]));
    const bool counts = (lane & 4) == 0;  // each (token, head) is held by two lanes; one of them counts
    v4f acc[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = (v4f){0.f, 0.f, 0.f, 0.f};
    float lsum = 0.0f, csum = 0.0f;
    auto pv = [&](const v4i &vv, float vscale, float score) {
        const float pe = __builtin_amdgcn_exp2f(score - m_h);   // masked tokens: exp2(-inf) = 0
        const float a = pe * vscale;
        if (counts) { lsum += pe; csum += a; }
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const uint32_t x = (uint32_t)vv[w] ^ 0x80808080u;
            acc[4 * w + 0] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, (float)(x & 0xffu), acc[4 * w + 0], 0, 0, 0);
            acc[4 * w + 1] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, (float)((x >> 8) & 0xffu), acc[4 * w + 1], 0, 0, 0);
            acc[4 * w + 2] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, (float)((x >> 16) & 0xffu), acc[4 * w + 2], 0, 0, 0);
            acc[4 * w + 3] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, (float)(x >> 24), acc[4 * w + 3], 0, 0, 0);
        }
    };
#pragma unroll
    for (int u = 0; u < WAVE_GROUPS / 2; ++u) pv(va[u], vsa[u], sc[u]);
#pragma unroll
    for (int u = 0; u < WAVE_GROUPS / 2; ++u) pv(vb[u], vsb2[u], sc[u + WAVE_GROUPS / 2]);

    // sum the 8 token slots (lanes that share l%8): transposed butterfly over lane bits 5, 4, 3, after which
    // lane l holds the 8 totals with flat index 8*(l/8) .. +7, flat = 4*e + head  (56 shuffles, not 192)
    float flat[64];
#pragma unroll
    for (int e = 0; e < 16; ++e)
#pragma unroll
        for (int i = 0; i < 4; ++i) flat[4 * e + i] = acc[e][i];
    fold_slots<64, 32>(flat, lane);
    fold_slots<32, 16>(flat, lane);
    fold_slots<16, 8>(flat, lane);
    lsum += slot_xor<8>(lsum); lsum += slot_xor<16>(lsum); lsum += slot_xor<32>(lsum);
    csum += slot_xor<8>(csum); csum += slot_xor<16>(csum); csum += slot_xor<32>(csum);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int fl = 8 * slot + j;   // = 4*e + head
        s_red[wave][fl & 3][16 * chunk + (fl >> 2)] = flat[j];
    }
    if (lane < 4) { s_l[wave][lane] = lsum; s_c[wave][lane] = csum; }
    __syncthreads();

    const int64_t pbase = ((int64_t)bkv * gridDim.x + split);
    for (int o = tid; o < 4 * D; o += 256) {
        const int h = o >> 7, d = o & (D - 1);
        const float c = s_c[0][h] + s_c[1][h] + s_c[2][h] + s_c[3][h];
        const float sum = s_red[0][h][d] + s_red[1][h][d] + s_red[2][h][d] + s_red[3][h][d];
        p.part_o[(pbase * 4 + h) * D + d] = sum - 128.0f * c;
    }
    if (tid < 4) {
        p.part_ml[pbase * 8 + tid] = fmaxf(fmaxf(s_m[0][tid], s_m[1][tid]), fmaxf(s_m[2][tid], s_m[3][tid]));
        p.part_ml[pbase * 8 + 4 + tid] = s_l[0][tid] + s_l[1][tid] + s_l[2][tid] + s_l[3][tid];
    }
}

// merge the splits of 16 (b, h) rows per workgroup; 16 lanes per row
__global__ __launch_bounds__(256) void k_gqa_merge(const float *__restrict__ part_o,
                                                   const float *__restrict__ part_ml, float *__restrict__ o,
                                                   int rows, int Hq, int Hkv, int G, int splits, int out_rotated)
{
    const int tid = threadIdx.x, j = tid & 15;
    const int row = blockIdx.x * 16 + (tid >> 4);
    const bool live = row < rows;
    const int rr = live ? row : rows - 1;
    const int b = rr / Hq, h = rr % Hq, kvh = h / G, hl = h % G;
    const int64_t bkv = (int64_t)b * Hkv + kvh;
    float mx = -INFINITY;
    for (int s = 0; s < splits; ++s) mx = fmaxf(mx, part_ml[(bkv * splits + s) * 8 + hl]);
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float l = 0.0f;
    for (int s = 0; s < splits; ++s) {
        const float *ml = part_ml + (bkv * splits + s) * 8;
        const float w = __builtin_amdgcn_exp2f(ml[hl] - mx);
        l = __builtin_fmaf(ml[4 + hl], w, l);
        const float *po = part_o + ((bkv * splits + s) * 4 + hl) * attn::D;
        const float4 lo = *reinterpret_cast<const float4 *>(po + 4 * j);
        const float4 hi = *reinterpret_cast<const float4 *>(po + 64 + 4 * j);
        v[0] = __builtin_fmaf(lo.x, w, v[0]); v[1] = __builtin_fmaf(lo.y, w, v[1]);
        v[2] = __builtin_fmaf(lo.z, w, v[2]); v[3] = __builtin_fmaf(lo.w, w, v[3]);
        v[4] = __builtin_fmaf(hi.x, w, v[4]); v[5] = __builtin_fmaf(hi.y, w, v[5]);
        v[6] = __builtin_fmaf(hi.z, w, v[6]); v[7] = __builtin_fmaf(hi.w, w, v[7]);
    }
    const float rl = 1.0f / l;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] *= rl;
    if (!out_rotated) fwht128(v, j);  // whole workgroup takes the same branch
    if (live) {
        float *orow = o + (int64_t)row * attn::D;
        *reinterpret_cast<float4 *>(orow + 4 * j) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4 *>(orow + 64 + 4 * j) = make_float4(v[4], v[5], v[6], v[7]);
    }
}

static int pick_splits(int64_t B, int64_t Hkv, int64_t T)
{
    const int ntiles = (int)((T + 15) / 16);
    const int cus = compute_units();
    constexpr int MAX_TILES = 4 * WAVE_GROUPS / 2;   // 16-token tiles one workgroup can hold in registers
    int splits = (ntiles + MAX_TILES - 1) / MAX_TILES;
    // short caches / few heads: more, shorter splits until there are about two workgroups per compute unit
    while (B * Hkv * splits < 2LL * cus && (ntiles + splits - 1) / splits > 8) splits *= 2;
    if (splits > ntiles) splits = ntiles;
    return splits;
}

static int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

}  // namespace attn
}  // namespace mi

using namespace mi;

static int32_t check_attn(int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T)
{
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || T <= 0) return MI_EINVAL;
    if (D != attn::D) return MI_EINVAL;
    if (Hq % Hkv || Hq / Hkv > 4) return MI_EINVAL;
    if (T > (1LL << 24) || B * Hkv > 65535) return MI_ERANGE;
    return MI_OK;
}

extern "C" int64_t mi_gqa_decode_workspace_bytes(int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T)
{
    int32_t rc = check_attn(B, Hq, Hkv, D, T);
    if (rc) return rc;
    const int splits = attn::pick_splits(B, Hkv, T);
    return attn::align_up(B * Hkv * splits * 4 * attn::D * 4, 256) + attn::align_up(B * Hkv * splits * 8 * 4, 256);
}

static int32_t run_attn(const float *q, const int8_t *kq, const float *ks, const int8_t *vq, const float *vs,
                        float *o, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T, int32_t out_rotated,
                        void *workspace, int64_t workspace_bytes, int8_t *dqq, float *dsq, int32_t *ddots,
                        hipStream_t s)
{
    int32_t rc = check_attn(B, Hq, Hkv, D, T);
    if (rc) return rc;
    if (!q || !kq || !ks || !vq || !vs || !workspace) return MI_EINVAL;
    if (!aligned16(q) || !aligned16(kq) || !aligned16(vq) || !aligned4(ks) || !aligned4(vs) || !aligned16(workspace))
        return MI_EINVAL;
    if (workspace_bytes < mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T)) return MI_ENOSPC;
    const int splits = attn::pick_splits(B, Hkv, T);
    const int ntiles = (int)((T + 15) / 16);
    attn::Params p;
    p.q = q; p.kq = kq; p.ks = ks; p.vq = vq; p.vs = vs;
    p.part_o = static_cast<float *>(workspace);
    p.part_ml = reinterpret_cast<float *>(static_cast<char *>(workspace) +
                                          attn::align_up(B * Hkv * splits * 4 * attn::D * 4, 256));
    p.dump_qq = dqq; p.dump_sq = dsq; p.dump_dots = ddots;
    p.Hq = (int)Hq; p.Hkv = (int)Hkv; p.G = (int)(Hq / Hkv); p.T = (int)T;
    p.tiles_per_split = (ntiles + splits - 1) / splits;
    p.score_scale = 1.4426950408889634f * 0.08838834764831845f;  // log2(e) / sqrt(128)
    const dim3 grid((unsigned)splits, (unsigned)(B * Hkv));
    if (ddots) hipLaunchKernelGGL(attn::k_gqa_split<true>, grid, dim3(256), 0, s, p);
    else hipLaunchKernelGGL(attn::k_gqa_split<false>, grid, dim3(256), 0, s, p);
    rc = launch_status();
    if (rc || !o) return rc;
    const int rows = (int)(B * Hq);
    hipLaunchKernelGGL(attn::k_gqa_merge, dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, s, p.part_o, p.part_ml, o,
                       rows, (int)Hq, (int)Hkv, p.G, splits, out_rotated);
    return launch_status();
}

extern "C" int32_t mi_gqa_decode_attn(const float *q, const int8_t *kq, const float *ks, const int8_t *vq,
                                      const float *vs, float *o, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                                      int64_t T, int32_t out_rotated, void *workspace, int64_t workspace_bytes,
                                      void *stream)
{
    if (!o || !aligned16(o)) return MI_EINVAL;
    return run_attn(q, kq, ks, vq, vs, o, B, Hq, Hkv, D, T, out_rotated, workspace, workspace_bytes, nullptr, nullptr,
                    nullptr, as_stream(stream));
}

extern "C" int32_t mi_gqa_decode_scores_i32(const float *q, const int8_t *kq, const float *ks, const int8_t *vq,
                                            const float *vs, int8_t *qq, float *sq, int32_t *dots, int64_t B,
                                            int64_t Hq, int64_t Hkv, int64_t D, int64_t T, void *workspace,
                                            int64_t workspace_bytes, void *stream)
{
    if (!qq || !sq || !dots || !aligned4(qq) || !aligned4(sq) || !aligned4(dots)) return MI_EINVAL;
    return run_attn(q, kq, ks, vq, vs, nullptr, B, Hq, Hkv, D, T, 1, workspace, workspace_bytes, qq, sq, dots,
                    as_stream(stream));
}
