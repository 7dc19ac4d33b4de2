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
// Pass 1 (scores).  Keys are loaded straight in MFMA operand layout (lane l: token l%16 of a 16-token tile,
// 16-byte chunk l/16 of each half of the head dimension); two v_mfma_i32_16x16x64_i8 per tile against the
// query codes of the G heads give the exact int32 dot products (lane l < 16: token l, register r: head r).
// Scores (already in log2 units) go to LDS, the running max stays in registers.
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
#include "fwht_core.h"

namespace mi {

namespace avt {
int max_splits(int64_t B, int64_t Hkv, int64_t T);   // attention_tiled.hip: the block-transposed V layout's own plan
}

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

__device__ __forceinline__ void fwht128(float (&v)[8], int j) { fwht_chunk<D>(v, j); }   // fwht_core.h

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
    int Hq, Hkv, G, T;    // T: tokens per sequence (the longest one when seq_len is given)
    int Tstride;          // tokens between consecutive (batch, kv head) rows of the cache
    const int32_t *seq_len;   // per-sequence token counts [B] (device), or null: every sequence holds T tokens
    const int32_t *block_table;   // paged cache: page of tokens [i*P, (i+1)*P) of sequence b at [b*max_pages + i], or null
    int max_pages, page_shift;    // P = 1 << page_shift tokens per page, P >= 16
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

// 16-token tiles per wave: a workgroup covers at most 4 * tiles * 16 tokens.  Every wave runs through all of its
// tiles (the ones past the end masked), so a workgroup wants a span it can fill: 11 tiles (704 tokens) when there
// are (batch, kv head) rows enough to occupy the chip with such spans, 4 tiles (256 tokens) when there are few rows
// and the cache has to be cut finer to give every compute unit work.
constexpr int TILES_LONG = 11, TILES_SHORT = 4;
constexpr int RING = 8;           // loads a wave keeps in flight (1 KB each); tiles per wave >= RING / 2

// RAGGED: the span a workgroup can cover runs past the end of the cache and token indices are clamped for the
// loads; otherwise every address is base + constant.  Tokens past the end of the split are masked in the scores.
// PAGED: the cache is a pool of pages [page][kv head][P tokens][128]; a 16-token tile lies in one page, so a wave
// looks up one page per tile (uniform over the wave) and lanes are clamped inside their tile.
template <bool DUMP, bool RAGGED, bool PAGED, int WAVE_TILES>
__device__ __forceinline__ void gqa_split_body(const Params &p, const int T, int8_t (&s_q)[4][4][D], float (&s_sq)[4][4],
                                               float (&s_red)[4][4][D], float (&s_sc)[4][WAVE_TILES][16][4],
                                               float (&s_m)[4][4], float (&s_l)[4][4], float (&s_c)[4][4])
{
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int split = blockIdx.x, bkv = blockIdx.y;
    const int b = bkv / p.Hkv, kvh = bkv % p.Hkv;
    const int G = p.G;
    const int ntiles = (T + 15) >> 4;
    const int tile_lo = split * p.tiles_per_split;
    const int tile_hi = min(tile_lo + p.tiles_per_split, ntiles);
    const int t_lo = tile_lo << 4;
    const int t_end = min(tile_hi << 4, T);   // first token this workgroup does not own
    // pass 1 lane layout (MFMA operand B): token l%16 of a 16-token tile, 16-byte chunk l/16 (+4 for the
    // second half of the head dimension); pass 2 lane layout: token slot l/8 of an 8-token group, chunk l%8
    const int tk16 = lane & 15, ck = lane >> 4;
    const int hh = lane & 3, slot = lane >> 3, chunk = lane & 7;
    const int t_wave = t_lo + wave * 16;      // first token of this wave's tile 0; tile j starts 64 tokens further
    const int8_t *kwave = p.kq + ((int64_t)bkv * p.Tstride + t_wave) * D;
    const int8_t *vwave = p.vq + ((int64_t)bkv * p.Tstride + t_wave) * D;
    const float *kswave = p.ks + (int64_t)bkv * p.Tstride + t_wave;
    const float *vswave = p.vs + (int64_t)bkv * p.Tstride + t_wave;
    const unsigned koff = (unsigned)(tk16 * D + 16 * ck);
    // paged: row index (in tokens) of the first token of each of the wave's tiles inside the pool, and the last
    // valid token offset inside that tile (tiles past the end of the sequence fall back on its last tile and are
    // masked in the scores like any token past the end)
    int64_t trow[PAGED ? WAVE_TILES : 1];
    int tlast[PAGED ? WAVE_TILES : 1];
    if constexpr (PAGED) {
        const int last_tile = (T - 1) & ~15;
#pragma unroll
        for (int j = 0; j < WAVE_TILES; ++j) {
            const int tt = min(t_wave + j * 64, last_tile);
            const int page = __builtin_amdgcn_readfirstlane(p.block_table[(int64_t)b * p.max_pages + (tt >> p.page_shift)]);
            trow[j] = (((int64_t)page * p.Hkv + kvh) << p.page_shift) + (tt & ((1 << p.page_shift) - 1));
            tlast[j] = min(T - 1 - tt, 15);
        }
    }

    // the query row goes first: loads return in order, and the rotation of q can then run under the key loads
    const int hr = lane >> 4, jj = lane & 15;
    const int head = kvh * G + min(hr, G - 1);
    const float *qr = p.q + ((int64_t)b * p.Hq + head) * D;
    const float4 qlo = *reinterpret_cast<const float4 *>(qr + 4 * jj);
    const float4 qhi = *reinterpret_cast<const float4 *>(qr + 64 + 4 * jj);

    // ---- the wave streams its 8 key tiles (two 1 KB loads each) and then its 16 value groups (one 1 KB load
    // each) through a ring of RING register slots.  A slot is refilled as soon as it has been consumed, so RING
    // KB stay in flight per wave from the first instruction to the last and the arithmetic runs under the stream.
    v4i ring[RING];
    float ksr[RING / 2], vsr[RING];
    auto load_k = [&](int j) {   // tile j -> slots (2j) % RING, (2j+1) % RING
        if constexpr (PAGED) {
            const int64_t row = trow[j] + min(tk16, tlast[j]);
            ring[(2 * j) % RING] = *reinterpret_cast<const v4i *>(p.kq + row * D + 16 * ck);
            ring[(2 * j + 1) % RING] = *reinterpret_cast<const v4i *>(p.kq + row * D + 64 + 16 * ck);
            ksr[j % (RING / 2)] = p.ks[row];
        } else if constexpr (RAGGED) {
            const int tk = min(t_wave + j * 64 + tk16, T - 1) - t_wave;
            ring[(2 * j) % RING] = *reinterpret_cast<const v4i *>(kwave + (int64_t)tk * D + 16 * ck);
            ring[(2 * j + 1) % RING] = *reinterpret_cast<const v4i *>(kwave + (int64_t)tk * D + 64 + 16 * ck);
            ksr[j % (RING / 2)] = kswave[tk];
        } else {
            ring[(2 * j) % RING] = *reinterpret_cast<const v4i *>(kwave + (koff + (unsigned)(j * 64 * D)));
            ring[(2 * j + 1) % RING] = *reinterpret_cast<const v4i *>(kwave + (koff + (unsigned)(j * 64 * D + 64)));
            ksr[j % (RING / 2)] = kswave[(unsigned)(j * 64) + (unsigned)tk16];
        }
    };
    auto load_v = [&](int u) {   // group u = 2*tile + half -> slot (2*WAVE_TILES + u) % RING
        const int j = u >> 1, g = u & 1;
        if constexpr (PAGED) {
            const int64_t row = trow[j] + min(g * 8 + slot, tlast[j]);
            ring[(2 * WAVE_TILES + u) % RING] = *reinterpret_cast<const v4i *>(p.vq + row * D + 16 * chunk);
            vsr[u % RING] = p.vs[row];
        } else if constexpr (RAGGED) {
            const int tk = min(t_wave + j * 64 + g * 8 + slot, T - 1) - t_wave;
            ring[(2 * WAVE_TILES + u) % RING] = *reinterpret_cast<const v4i *>(vwave + (int64_t)tk * D + 16 * chunk);
            vsr[u % RING] = vswave[tk];
        } else {
            ring[(2 * WAVE_TILES + u) % RING] =
                *reinterpret_cast<const v4i *>(vwave + ((unsigned)(lane * 16) + (unsigned)(j * 64 * D + g * 8 * D)));
            vsr[u % RING] = vswave[(unsigned)(j * 64 + g * 8) + (unsigned)slot];
        }
    };
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < RING / 2; ++j) load_k(j);
    __builtin_amdgcn_sched_barrier(0);

    // ---- query heads of this group: every wave rotates and quantizes them for itself (no workgroup barrier)
    {
        float v[8] = {qlo.x, qlo.y, qlo.z, qlo.w, qhi.x, qhi.y, qhi.z, qhi.w};
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
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // MFMA operand A: row l%16 = query head (rows >= G are zero), 16-byte chunk l/16 (+4)
    v4i qa0 = {0, 0, 0, 0}, qa1 = {0, 0, 0, 0};
    if (tk16 < G) {
        qa0 = *reinterpret_cast<const v4i *>(&s_q[wave][tk16][16 * ck]);
        qa1 = *reinterpret_cast<const v4i *>(&s_q[wave][tk16][64 + 16 * ck]);
    }
    float cq[4];     // per-head factor of the score, log2 units
#pragma unroll
    for (int h = 0; h < 4; ++h) cq[h] = h < G ? s_sq[wave][h] * p.score_scale : 0.0f;

    // ---- pass 1: scores.  Two v_mfma_i32_16x16x64_i8 per tile give the exact int32 dot products of the 16
    // tokens with the G heads; lane l < 16 holds token l, register r = head r.  Scores (log2 units) go to LDS.
    float m4[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
    for (int j = 0; j < WAVE_TILES; ++j) {
        v4i dots = __builtin_amdgcn_mfma_i32_16x16x64_i8(qa0, ring[(2 * j) % RING], (v4i){0, 0, 0, 0}, 0, 0, 0);
        dots = __builtin_amdgcn_mfma_i32_16x16x64_i8(qa1, ring[(2 * j + 1) % RING], dots, 0, 0, 0);
        const float kscale = ksr[j % (RING / 2)];
        // the two slots are free: next key tile, or the first value groups once the keys are all requested
        if (j + RING / 2 < WAVE_TILES) load_k(j + RING / 2);
        else { load_v(2 * (j + RING / 2 - WAVE_TILES)); load_v(2 * (j + RING / 2 - WAVE_TILES) + 1); }
        __builtin_amdgcn_sched_barrier(0);
        const int tt = t_wave + j * 64 + tk16;
        const bool live = tt < t_end;
        float4 sc;
        sc.x = live ? (float)dots[0] * (kscale * cq[0]) : -INFINITY;
        sc.y = live ? (float)dots[1] * (kscale * cq[1]) : -INFINITY;
        sc.z = live ? (float)dots[2] * (kscale * cq[2]) : -INFINITY;
        sc.w = live ? (float)dots[3] * (kscale * cq[3]) : -INFINITY;
        if (lane < 16) {
            *reinterpret_cast<float4 *>(&s_sc[wave][j][tk16][0]) = sc;
            m4[0] = fmaxf(m4[0], sc.x); m4[1] = fmaxf(m4[1], sc.y);
            m4[2] = fmaxf(m4[2], sc.z); m4[3] = fmaxf(m4[3], sc.w);
            if constexpr (DUMP) {
                if (live) {
#pragma unroll
                    for (int h = 0; h < 4; ++h)
                        if (h < G) p.dump_dots[((int64_t)b * p.Hq + kvh * G + h) * T + tt] = dots[h];
                }
            }
        }
    }
    // maximum per head over the wave's tokens (lanes 0..15 hold partial maxima, the rest hold -inf); the softmax
    // of this wave is taken against the wave's own maximum and rescaled when the waves meet
#pragma unroll
    for (int h = 0; h < 4; ++h) {
        m4[h] = fmaxf(m4[h], lane_xor<1>(m4[h]));
        m4[h] = fmaxf(m4[h], lane_xor<2>(m4[h]));
        m4[h] = fmaxf(m4[h], lane_xor<4>(m4[h]));
        m4[h] = fmaxf(m4[h], lane_xor<8>(m4[h]));
    }
    if (lane == 0) { s_m[wave][0] = m4[0]; s_m[wave][1] = m4[1]; s_m[wave][2] = m4[2]; s_m[wave][3] = m4[3]; }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const float m_h = s_m[wave][hh];

    // ---- pass 2: P.V on the fp32 matrix pipe
    const bool counts = (lane & 4) == 0;  // each (token, head) is held by two lanes; one of them counts
    v4f acc[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = (v4f){0.f, 0.f, 0.f, 0.f};
    float lsum = 0.0f, csum = 0.0f;
#pragma unroll
    for (int u = 0; u < 2 * WAVE_TILES; ++u) {
        const v4i vv = ring[(2 * WAVE_TILES + u) % RING];
        const float vscale = vsr[u % RING];
        // int8 -> fp32 as (byte ^ 0x80) - 128: v_cvt_f32_ubyteN on the biased byte, the bias leaves at the end
        float f[16];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const uint32_t x = (uint32_t)vv[w] ^ 0x80808080u;
            f[4 * w + 0] = (float)(x & 0xffu);
            f[4 * w + 1] = (float)((x >> 8) & 0xffu);
            f[4 * w + 2] = (float)((x >> 16) & 0xffu);
            f[4 * w + 3] = (float)(x >> 24);
        }
        if (u + RING < 2 * WAVE_TILES) load_v(u + RING);
        __builtin_amdgcn_sched_barrier(0);
        const float score = s_sc[wave][u >> 1][8 * (u & 1) + slot][hh];
        // a wave whose tokens are all masked has m_h = -inf: exp2(-inf - -inf) would be NaN
        const float pe = (score == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(score - m_h);
        const float a = pe * vscale;
        if (counts) { lsum += pe; csum += a; }
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[e] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, f[e], acc[e], 0, 0, 0);
    }

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

    // the four waves meet: rescale each wave's sums from its own maximum to the common one
    const int64_t pbase = ((int64_t)bkv * gridDim.x + split);
    for (int o = tid; o < 4 * D; o += 256) {
        const int h = o >> 7, d = o & (D - 1);
        const float m = fmaxf(fmaxf(s_m[0][h], s_m[1][h]), fmaxf(s_m[2][h], s_m[3][h]));
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float f = (s_m[w][h] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(s_m[w][h] - m);
            sum += (s_red[w][h][d] - 128.0f * s_c[w][h]) * f;
        }
        p.part_o[(pbase * 4 + h) * D + d] = sum;
    }
    if (tid < 4) {
        const float m = fmaxf(fmaxf(s_m[0][tid], s_m[1][tid]), fmaxf(s_m[2][tid], s_m[3][tid]));
        float l = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) l += (s_m[w][tid] == -INFINITY) ? 0.0f : s_l[w][tid] * __builtin_amdgcn_exp2f(s_m[w][tid] - m);
        p.part_ml[pbase * 8 + tid] = m;
        p.part_ml[pbase * 8 + 4 + tid] = l;
    }
}

template <bool DUMP, int WAVE_TILES>
__global__ __launch_bounds__(256) void k_gqa_split(Params p)
{
    __shared__ __attribute__((aligned(16))) int8_t s_q[4][4][D];
    __shared__ float s_sq[4][4];
    __shared__ float s_red[4][4][D];
    __shared__ __attribute__((aligned(16))) float s_sc[4][WAVE_TILES][16][4];
    __shared__ float s_m[4][4], s_l[4][4], s_c[4][4];
    const int tile_lo = blockIdx.x * p.tiles_per_split;
    int T = p.T;
    if (p.seq_len) {
        // a cache that is filled to a different length per sequence: lengths outside [0, T] are clamped
        const int b = blockIdx.y / p.Hkv;
        T = min(max(__builtin_amdgcn_readfirstlane(p.seq_len[b]), 0), p.T);
        if (tile_lo * 16 >= T) {
            // this split lies past the end of the sequence: an empty partial (weight 0 in the merge)
            const int64_t pbase = ((int64_t)blockIdx.y * gridDim.x + blockIdx.x);
            for (int o = threadIdx.x; o < 4 * D; o += 256) p.part_o[pbase * 4 * D + o] = 0.0f;
            if (threadIdx.x < 4) {
                p.part_ml[pbase * 8 + threadIdx.x] = -INFINITY;
                p.part_ml[pbase * 8 + 4 + threadIdx.x] = 0.0f;
            }
            return;
        }
    }
    if (p.block_table) {
        gqa_split_body<false, true, true, WAVE_TILES>(p, T, s_q, s_sq, s_red, s_sc, s_m, s_l, s_c);
        return;
    }
    const bool full = (tile_lo + 4 * WAVE_TILES) * 16 <= T;
    if (full) gqa_split_body<DUMP, false, false, WAVE_TILES>(p, T, s_q, s_sq, s_red, s_sc, s_m, s_l, s_c);
    else gqa_split_body<DUMP, true, false, WAVE_TILES>(p, T, s_q, s_sq, s_red, s_sc, s_m, s_l, s_c);
}

// Merge of the splits of one (b, h) row by the 16 lanes that own it (lane j: elements 4j..4j+3 and 64+4j..).
// SP > 0: the split count is known at compile time and every load of the row goes out before the first use (one
// memory round trip).  Returns the normalized row in the rotated basis of V.
template <int SP, int BATCH = 8>
__device__ __forceinline__ void merge_row(const float *__restrict__ part_o, const float *__restrict__ part_ml,
                                          int splits_rt, int64_t bkv, int hl, int j, float (&v)[8])
{
    const int splits = SP > 0 ? SP : splits_rt;
    const float *ml0 = part_ml + bkv * splits * 8;
    const float *po0 = part_o + (bkv * splits * 4 + hl) * attn::D;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = 0.0f;
    float l = 0.0f;
    if constexpr (SP > 0) {
        float ms[SP], ls[SP];
        float4 lo[SP], hi[SP];
#pragma unroll
        for (int s = 0; s < SP; ++s) {
            ms[s] = ml0[s * 8 + hl];
            ls[s] = ml0[s * 8 + 4 + hl];
            lo[s] = *reinterpret_cast<const float4 *>(po0 + s * 4 * attn::D + 4 * j);
            hi[s] = *reinterpret_cast<const float4 *>(po0 + s * 4 * attn::D + 64 + 4 * j);
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
    } else {
        // any split count: the maxima first (one round trip), then the partials in batches of BATCH whose loads all
        // go out before the first use
        float mx = -INFINITY;
        for (int s0 = 0; s0 < splits; s0 += BATCH) {
            float ms[BATCH];
#pragma unroll
            for (int i = 0; i < BATCH; ++i) ms[i] = ml0[min(s0 + i, splits - 1) * 8 + hl];
#pragma unroll
            for (int i = 0; i < BATCH; ++i) mx = fmaxf(mx, ms[i]);
        }
        for (int s0 = 0; s0 < splits; s0 += BATCH) {
            float ms[BATCH], ls[BATCH];
            float4 lo[BATCH], hi[BATCH];
#pragma unroll
            for (int i = 0; i < BATCH; ++i) {
                const int s = min(s0 + i, splits - 1);
                ms[i] = ml0[s * 8 + hl];
                ls[i] = ml0[s * 8 + 4 + hl];
                lo[i] = *reinterpret_cast<const float4 *>(po0 + s * 4 * attn::D + 4 * j);
                hi[i] = *reinterpret_cast<const float4 *>(po0 + s * 4 * attn::D + 64 + 4 * j);
            }
#pragma unroll
            for (int i = 0; i < BATCH; ++i) {
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

// merge the splits of blockDim.x / 16 (b, h) rows per workgroup; 16 lanes per row.  Few rows with many splits (one
// token) take one row per workgroup, so that no compute unit reads more than one row's partials.
template <int SP>
__global__ __launch_bounds__(256) void k_gqa_merge(const float *__restrict__ part_o,
                                                   const float *__restrict__ part_ml, float *__restrict__ o,
                                                   int rows, int Hq, int Hkv, int G, int splits_rt, int out_rotated)
{
    const int tid = threadIdx.x, j = tid & 15;
    const int row = blockIdx.x * (int)(blockDim.x >> 4) + (tid >> 4);
    const bool live = row < rows;
    const int rr = live ? row : rows - 1;
    const int b = rr / Hq, h = rr % Hq, kvh = h / G, hl = h % G;
    const int64_t bkv = (int64_t)b * Hkv + kvh;
    float v[8];
    merge_row<SP, 16>(part_o, part_ml, splits_rt, bkv, hl, j, v);
    if (!out_rotated) fwht128(v, j);  // whole workgroup takes the same branch
    if (live) {
        float *orow = o + (int64_t)row * attn::D;
        *reinterpret_cast<float4 *>(orow + 4 * j) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4 *>(orow + 64 + 4 * j) = make_float4(v[4], v[5], v[6], v[7]);
    }
}

// Rows that were cut into 17 .. 32 splits (one or two tokens over a long cache): 32 lanes per row, one float4 per lane
// and split, and every load of the row in flight at once.  The partials were written by workgroups all over the
// chip, so every dependent batch of loads is a round trip to memory of 2-3 us: merge_row's batches of 8 or 16 cost
// four of them here, this kernel one.  Per element the sum runs over the splits in index order with the same
// operations as merge_row: the same bits.
__global__ __launch_bounds__(64) void k_gqa_merge_wide(const float *__restrict__ part_o,
                                                       const float *__restrict__ part_ml, float *__restrict__ o,
                                                       int rows, int Hq, int Hkv, int G, int splits, int out_rotated)
{
    constexpr int SMAX = 32;
    const int tid = threadIdx.x, j = tid & 15, half = (tid >> 4) & 1;
    const int row = blockIdx.x * 2 + (tid >> 5);
    const bool live = row < rows;
    const int rr = live ? row : rows - 1;
    const int b = rr / Hq, h = rr % Hq, kvh = h / G, hl = h % G;
    const int64_t bkv = (int64_t)b * Hkv + kvh;
    const float *ml0 = part_ml + bkv * splits * 8;
    const float *po0 = part_o + (bkv * splits * 4 + hl) * attn::D + half * 64 + 4 * j;
    float ms[SMAX], ls[SMAX];
    float4 d[SMAX];
#pragma unroll
    for (int s = 0; s < SMAX; ++s) {
        const int sc = min(s, splits - 1);
        ms[s] = ml0[sc * 8 + hl];
        ls[s] = ml0[sc * 8 + 4 + hl];
        d[s] = *reinterpret_cast<const float4 *>(po0 + sc * 4 * attn::D);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int s = 0; s < SMAX; ++s) mx = fmaxf(mx, ms[s]);
    float l = 0.0f, v0 = 0.0f, v1 = 0.0f, v2 = 0.0f, v3 = 0.0f;
#pragma unroll
    for (int s = 0; s < SMAX; ++s) {
        const float w = (s >= splits || ms[s] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(ms[s] - mx);
        l = __builtin_fmaf(ls[s], w, l);
        v0 = __builtin_fmaf(d[s].x, w, v0); v1 = __builtin_fmaf(d[s].y, w, v1);
        v2 = __builtin_fmaf(d[s].z, w, v2); v3 = __builtin_fmaf(d[s].w, w, v3);
    }
    const float rl = l > 0.0f ? 1.0f / l : 0.0f;
    v0 *= rl; v1 *= rl; v2 *= rl; v3 *= rl;
    float *orow = o + (int64_t)row * attn::D;
    if (out_rotated) {
        if (live) *reinterpret_cast<float4 *>(orow + half * 64 + 4 * j) = make_float4(v0, v1, v2, v3);
        return;
    }
    // inverse rotation: the lower 16 lanes of a row collect the upper 16 lanes' elements 64 + 4j .. and run the
    // 16-lane butterfly (the upper lanes run it too, on their own values twice, and store nothing)
    const int src = (tid & ~31) | (16 + j);
    float v[8] = {v0, v1, v2, v3, __shfl(v0, src, 64), __shfl(v1, src, 64), __shfl(v2, src, 64), __shfl(v3, src, 64)};
    fwht128(v, j);
    if (live && half == 0) {
        *reinterpret_cast<float4 *>(orow + 4 * j) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4 *>(orow + 64 + 4 * j) = make_float4(v[4], v[5], v[6], v[7]);
    }
}

// The merge of one token's Hq rows by one workgroup (16 lanes per head), followed by the int8 row quantizer over the
// token's Hq*128 values as they stand in the rotated basis of V: the codes and the scale are what the output
// projection's GEMV consumes when its weights were rotated along K with block 128 (x.H . (W.H)^T = x . W^T), so no
// inverse rotation and no second rotation are spent.  o_rot (optional) receives the fp32 row.
template <int SP>
__global__ __launch_bounds__(1024) void k_gqa_merge_quant(const float *__restrict__ part_o,
                                                          const float *__restrict__ part_ml,
                                                          float *__restrict__ o_rot, int8_t *__restrict__ oq,
                                                          float *__restrict__ oscale, int Hq, int Hkv, int G,
                                                          int splits_rt)
{
    __shared__ float s_max[16];
    const int tid = threadIdx.x, j = tid & 15, lane = tid & 63, wave = tid >> 6;
    const int b = blockIdx.x, h = tid >> 4;
    const int kvh = h / G, hl = h % G;
    float v[8];
    merge_row<SP>(part_o, part_ml, splits_rt, (int64_t)b * Hkv + kvh, hl, j, v);
    float a = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) a = fmaxf(a, fabsf(v[e]));
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) a = fmaxf(a, __shfl_xor(a, off, 64));
    if (lane == 0) s_max[wave] = a;
    __syncthreads();
    const int nwave = (int)(blockDim.x >> 6);
    a = s_max[0];
    for (int w = 1; w < nwave; ++w) a = fmaxf(a, s_max[w]);
    const float sc = (a == 0.0f) ? 1.0f : a / 127.0f;
    const float inv = (a == 0.0f) ? 0.0f : 127.0f / a;
    const int64_t off = ((int64_t)b * Hq + h) * attn::D;
    if (tid == 0) oscale[b] = sc;
    *reinterpret_cast<uint32_t *>(oq + off + 4 * j) = quant4(v[0], v[1], v[2], v[3], inv);
    *reinterpret_cast<uint32_t *>(oq + off + 64 + 4 * j) = quant4(v[4], v[5], v[6], v[7], inv);
    if (o_rot) {
        *reinterpret_cast<float4 *>(o_rot + off + 4 * j) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4 *>(o_rot + off + 64 + 4 * j) = make_float4(v[4], v[5], v[6], v[7]);
    }
}

struct SplitPlan {
    int splits, wave_tiles;
};

static SplitPlan pick_splits(int64_t B, int64_t Hkv, int64_t T)
{
    const int ntiles = (int)((T + 15) / 16);
    const int cus = compute_units();
    SplitPlan pl;
    pl.wave_tiles = TILES_LONG;
    pl.splits = (ntiles + 4 * TILES_LONG - 1) / (4 * TILES_LONG);
    if (B * Hkv * pl.splits < cus && ntiles > 4 * TILES_SHORT) {
        // few rows: spans of 256 tokens, then halves of them while that still doubles the number of busy compute units
        pl.wave_tiles = TILES_SHORT;
        pl.splits = (ntiles + 4 * TILES_SHORT - 1) / (4 * TILES_SHORT);
        while (B * Hkv * pl.splits < cus && (ntiles + pl.splits - 1) / pl.splits > 8 && pl.splits * 2 <= 16) pl.splits *= 2;
    }
    if (pl.splits > ntiles) pl.splits = ntiles;
    return pl;
}

// the largest split count pick_splits returns for any length in [1, T]
static int max_splits(int64_t B, int64_t Hkv, int64_t T)
{
    const int ntiles = (int)((T + 15) / 16);
    int best = (ntiles + 4 * TILES_LONG - 1) / (4 * TILES_LONG);   // long spans: monotone in T
    if (B * Hkv < compute_units()) {
        // short spans are possible for some length: ceil(n / 16) splits, doubled at most up to 16
        int s = (ntiles + 4 * TILES_SHORT - 1) / (4 * TILES_SHORT);
        if (s < 16) s = 16;
        if (s > ntiles) s = ntiles;
        if (s > best) best = s;
    }
    return best;
}

// Merge of the splits' partial results [B*Hkv, splits, 4, 128] / [B*Hkv, splits, 2, 4].  oq: one workgroup per token
// merges its Hq rows and quantizes them for the output projection (o then optionally receives the fp32 row in the
// rotated basis); otherwise 16 rows per workgroup into o.
int32_t launch_merge(const float *part_o, const float *part_ml, float *o, int8_t *oq, float *oscale, int64_t B,
                     int64_t Hq, int64_t Hkv, int splits, int out_rotated, hipStream_t s)
{
    const int G = (int)(Hq / Hkv);
    if (oq) {
#define MI_MERGEQ(SP)                                                                                           \
    hipLaunchKernelGGL(k_gqa_merge_quant<SP>, dim3((unsigned)B), dim3((unsigned)(Hq * 16)), 0, s, part_o, part_ml, \
                       o, oq, oscale, (int)Hq, (int)Hkv, G, splits)
        switch (splits) {
        case 1: MI_MERGEQ(1); break;
        case 2: MI_MERGEQ(2); break;
        case 4: MI_MERGEQ(4); break;
        case 6: MI_MERGEQ(6); break;
        case 8: MI_MERGEQ(8); break;
        case 12: MI_MERGEQ(12); break;
        case 16: MI_MERGEQ(16); break;
        default: MI_MERGEQ(0); break;
        }
#undef MI_MERGEQ
        return launch_status();
    }
    const int rows = (int)(B * Hq);
    if (splits > 16 && splits <= 32 && rows <= 2 * compute_units()) {
        hipLaunchKernelGGL(k_gqa_merge_wide, dim3((unsigned)((rows + 1) / 2)), dim3(64), 0, s, part_o, part_ml, o, rows,
                           (int)Hq, (int)Hkv, G, splits, out_rotated);
        return launch_status();
    }
    int rpw = 16;   // rows per workgroup: fewer while that still adds workgroups below half a chip's worth
    while (rpw > 1 && rows / rpw < compute_units() / 2) rpw >>= 1;
    const dim3 mgrid((unsigned)((rows + rpw - 1) / rpw)), mblock((unsigned)(16 * rpw));
#define MI_MERGE(SP)                                                                                              \
    hipLaunchKernelGGL(k_gqa_merge<SP>, mgrid, mblock, 0, s, part_o, part_ml, o, rows, (int)Hq, (int)Hkv, G, \
                       splits, out_rotated)
    switch (splits) {
    case 1: MI_MERGE(1); break;
    case 2: MI_MERGE(2); break;
    case 4: MI_MERGE(4); break;
    case 6: MI_MERGE(6); break;
    case 8: MI_MERGE(8); break;
    case 12: MI_MERGE(12); break;
    case 16: MI_MERGE(16); break;
    default: MI_MERGE(0); break;
    }
#undef MI_MERGE
    return launch_status();
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
    // an upper bound over every length up to T, so that a workspace sized for the capacity of a cache serves every
    // decode step: the plan is not monotone in T (a shorter sequence may be cut into more, shorter spans)
    int splits = attn::max_splits(B, Hkv, T);
    const int splits_vt = avt::max_splits(B, Hkv, T);   // one query serves both cache layouts
    if (splits_vt > splits) splits = splits_vt;
    return attn::align_up(B * Hkv * splits * 4 * attn::D * 4, 256) + attn::align_up(B * Hkv * splits * 8 * 4, 256);
}

static int32_t run_attn(const float *q, const int8_t *kq, const float *ks, const int8_t *vq, const float *vs,
                        float *o, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T, int32_t out_rotated,
                        void *workspace, int64_t workspace_bytes, int8_t *dqq, float *dsq, int32_t *ddots,
                        hipStream_t s, int64_t Tstride = 0, const int32_t *seq_len = nullptr, int8_t *oq = nullptr,
                        float *oscale = nullptr, const int32_t *block_table = nullptr, int64_t max_pages = 0,
                        int page_shift = 0)
{
    int32_t rc = check_attn(B, Hq, Hkv, D, T);
    if (rc) return rc;
    if (!q || !kq || !ks || !vq || !vs || !workspace) return MI_EINVAL;
    if (!aligned16(q) || !aligned16(kq) || !aligned16(vq) || !aligned4(ks) || !aligned4(vs) || !aligned16(workspace))
        return MI_EINVAL;
    if (workspace_bytes < mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T)) return MI_ENOSPC;
    const attn::SplitPlan plan = attn::pick_splits(B, Hkv, T);
    const int splits = plan.splits;
    const int ntiles = (int)((T + 15) / 16);
    attn::Params p;
    p.q = q; p.kq = kq; p.ks = ks; p.vq = vq; p.vs = vs;
    p.part_o = static_cast<float *>(workspace);
    p.part_ml = reinterpret_cast<float *>(static_cast<char *>(workspace) +
                                          attn::align_up(B * Hkv * splits * 4 * attn::D * 4, 256));
    p.dump_qq = dqq; p.dump_sq = dsq; p.dump_dots = ddots;
    p.Hq = (int)Hq; p.Hkv = (int)Hkv; p.G = (int)(Hq / Hkv); p.T = (int)T;
    p.Tstride = (int)(Tstride > 0 ? Tstride : T);
    p.seq_len = seq_len;
    p.block_table = block_table; p.max_pages = (int)max_pages; p.page_shift = page_shift;
    p.tiles_per_split = (ntiles + splits - 1) / splits;
    p.score_scale = 1.4426950408889634f * 0.08838834764831845f;  // log2(e) / sqrt(128)
    const dim3 grid((unsigned)splits, (unsigned)(B * Hkv));
    if (plan.wave_tiles == attn::TILES_LONG) {
        if (ddots) hipLaunchKernelGGL((attn::k_gqa_split<true, attn::TILES_LONG>), grid, dim3(256), 0, s, p);
        else hipLaunchKernelGGL((attn::k_gqa_split<false, attn::TILES_LONG>), grid, dim3(256), 0, s, p);
    } else {
        if (ddots) hipLaunchKernelGGL((attn::k_gqa_split<true, attn::TILES_SHORT>), grid, dim3(256), 0, s, p);
        else hipLaunchKernelGGL((attn::k_gqa_split<false, attn::TILES_SHORT>), grid, dim3(256), 0, s, p);
    }
    rc = launch_status();
    if (rc) return rc;
    if (!o && !oq) return rc;
    return attn::launch_merge(p.part_o, p.part_ml, o, oq, oscale, B, Hq, Hkv, splits, out_rotated, s);
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

extern "C" int32_t mi_gqa_decode_attn_cache(const float *q, const int8_t *kq, const float *ks, const int8_t *vq,
                                            const float *vs, float *o, int64_t B, int64_t Hq, int64_t Hkv,
                                            int64_t D, int64_t T_cap, const int32_t *seq_len, int64_t T_max,
                                            int32_t out_rotated, void *workspace, int64_t workspace_bytes,
                                            void *stream)
{
    if (!o || !aligned16(o) || !seq_len || !aligned4(seq_len)) return MI_EINVAL;
    if (T_cap <= 0 || T_max <= 0 || T_max > T_cap) return MI_EINVAL;
    if (T_cap > (1LL << 24)) return MI_ERANGE;
    return run_attn(q, kq, ks, vq, vs, o, B, Hq, Hkv, D, T_max, out_rotated, workspace, workspace_bytes, nullptr,
                    nullptr, nullptr, as_stream(stream), T_cap, seq_len);
}

extern "C" int32_t mi_gqa_decode_attn_cache_quant_i8(const float *q, const int8_t *kq, const float *ks,
                                                     const int8_t *vq, const float *vs, float *o_rot, int8_t *oq,
                                                     float *oscale, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                                                     int64_t T_cap, const int32_t *seq_len, int64_t T_max,
                                                     void *workspace, int64_t workspace_bytes, void *stream)
{
    if (!oq || !oscale || !aligned4(oq) || !aligned4(oscale) || (o_rot && !aligned16(o_rot))) return MI_EINVAL;
    if (!seq_len || !aligned4(seq_len)) return MI_EINVAL;
    if (T_cap <= 0 || T_max <= 0 || T_max > T_cap) return MI_EINVAL;
    if (T_cap > (1LL << 24) || Hq > 64) return MI_ERANGE;
    return run_attn(q, kq, ks, vq, vs, o_rot, B, Hq, Hkv, D, T_max, 1, workspace, workspace_bytes, nullptr, nullptr,
                    nullptr, as_stream(stream), T_cap, seq_len, oq, oscale);
}

extern "C" int32_t mi_gqa_decode_attn_paged(const float *q, const int8_t *kq_pool, const float *ks_pool,
                                            const int8_t *vq_pool, const float *vs_pool, float *o,
                                            const int32_t *block_table, int64_t max_pages, int64_t page_size,
                                            int64_t B, int64_t Hq, int64_t Hkv, int64_t D, const int32_t *seq_len,
                                            int64_t T_max, int32_t out_rotated, void *workspace,
                                            int64_t workspace_bytes, void *stream)
{
    if (!o || !aligned16(o) || !seq_len || !aligned4(seq_len) || !block_table || !aligned4(block_table))
        return MI_EINVAL;
    if (page_size < 16 || (page_size & (page_size - 1)) || page_size > (1 << 20)) return MI_EINVAL;
    if (T_max <= 0 || max_pages <= 0 || T_max > max_pages * page_size) return MI_EINVAL;
    if (max_pages > (1LL << 24)) return MI_ERANGE;
    int shift = 0;
    while ((1LL << shift) < page_size) ++shift;
    return run_attn(q, kq_pool, ks_pool, vq_pool, vs_pool, o, B, Hq, Hkv, D, T_max, out_rotated, workspace,
                    workspace_bytes, nullptr, nullptr, nullptr, as_stream(stream), 0, seq_len, nullptr, nullptr,
                    block_table, max_pages, shift);
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
