// Grouped-query decode attention over an int8 KV cache stored in the layouts the int8 matrix instruction loads
// straight from memory, 1 KB contiguous per wave instruction:
//   kt int8 [B, Hkv, T_cap/16, 8, 16, 16]  (tile of 16 tokens; byte (c, t % 16, e) = code 16*c + e of token t)
//   vt int8 [B, Hkv, T_cap/64, 8, 4, 16, 16]  (block of 64 tokens, transposed and cut into 16 x 16 pieces;
//                                           byte (d / 16, (t % 64) / 16, d % 16, t % 16) = code d of token t)
// A key load in operand layout (lane l: token l%16, 16-byte chunk l/16) is then lanes 0..63 reading consecutive
// 16-byte pieces, where the row-major cache [T, 128] makes the same load touch 16 lines of 128 bytes by halves.
// With tokens contiguous per head-dim row, a 16-byte load is 16 tokens of one output column, which is what the
// int8 matrix instruction wants for the contraction over tokens.  Both products of the attention then run on
// v_mfma_i32_16x16x64_i8 and no V byte is ever converted on the vector pipe:
//
//   scores   dots[t, h] = sum_d kq[t, d] * qq[h, d]          A = 16 tokens x 64 d, B = 64 d x 16 (G heads used)
//   P.V      o[h, d]    = sum_t p[t, h] * vs[t] * vq[t, d]   A = 16 rows x 64 tokens, B = a vt piece (64 t x 16 d)
//
// For the second product the fp32 weights a[t, h] = exp2(s[t, h] - m[h]) * vs[t] are written as fixed-point
// numbers of 28 bits relative to the largest V scale of the workgroup's span (rounded to nearest: a token whose V
// scale is 1/r of that largest one keeps 28 - log2(r) bits of its weight, more than fp32's 24 while r < 16) and
// cut into four 7-bit digits; digit k of head h is row 4*k + h of A, so that ONE instruction multiplies all four
// digits of the four heads with the block, and the four int32 partial sums are recombined in fp32 when the wave is
// done.  Inside a wave the sums are exact integers (any order), across waves and splits fp32 as before.
//
// A workgroup of four waves owns one span of 64-token blocks of one (batch, kv head) row; wave w takes blocks
// w, w + 4, ... of it.  Pass 1 streams the wave's key blocks (8 loads of 1 KB each) and leaves the scores in LDS;
// pass 2 streams the value blocks.  All loads run through one ring of register slots that is refilled slot by slot,
// keys first, values behind them, so that the same number of bytes stays in flight from the first instruction to
// the last.  The per-token scales of the span are staged in LDS once, up front.
//
// The partial results have the layout the merge kernels of attention.hip take.
//
// Bound: HBM (the K and V codes, 2 * B * Hkv * T * 128 bytes, + 8 bytes of scales per token-head).
#include "fwht_core.h"

namespace mi {
namespace attn {
int32_t launch_merge(const float *part_o, const float *part_ml, float *o, int8_t *oq, float *oscale, int64_t B,
                     int64_t Hq, int64_t Hkv, int splits, int out_rotated, hipStream_t s);
}
namespace avt {

constexpr int D = 128;
constexpr int SROW = 64 + 16;                // floats per (head, block) score row: rows 64 bytes apart modulo the
                                             // 256 bytes an LDS cycle serves, so that the 16 lanes of a group hit
                                             // 16 distinct 16-byte slots in both passes
constexpr float FIX_ONE = 268435200.0f;      // 2^28 - 256: the fixed-point image of the largest weight

struct Params {
    const float *q;
    const int8_t *kq;
    const float *ks;
    const int8_t *vt;
    const float *vs;
    float *part_o;    // [B*Hkv, splits, 4, 128]
    float *part_ml;   // [B*Hkv, splits, 2, 4]   (max in log2 units, sum)
    int Hq, Hkv, G, T;
    int Tstride;              // tokens between consecutive (batch, kv head) rows of the cache, a multiple of 64
    const int32_t *seq_len;   // per-sequence token counts [B] (device), or null: every sequence holds T tokens
    int blocks_per_split;     // 64-token blocks per workgroup, <= NW * NT
    float score_scale;        // log2(e) / sqrt(D)
    float *o;                 // DIRECT kernels: the output rows [B, Hq, 128]
    int out_rotated;
    // paged cache: kq / vt are pools of 8 KB blocks [page][kv head], ks / vs pools of 64 scales [page][kv head];
    // 64-token block i of sequence b lives in page block_table[b * max_pages + i].  Null: the dense layout.
    const int32_t *block_table;
    int max_pages;
    // gate outputs (null in production): the int8 query codes [B, Hq, 128], their scales [B, Hq] and the raw int32
    // dots [B, Hq, T] this kernel works from
    int8_t *dbg_qq;
    float *dbg_sq;
    int32_t *dbg_dots;
};

template <int MASK>
__device__ __forceinline__ float fmax_xor(float v)
{
    return fmaxf(v, xor_lane<MASK>(v));
}

// NW: waves per workgroup; NT: blocks per wave; RING: 1 KB loads a wave keeps in flight (8 or 16).
// DIRECT: the workgroup covers the whole sequence (one split): it normalizes and writes the output rows itself and
// no partial result leaves the chip.
template <int NW, int NT, int RING, bool DIRECT>
__global__ __launch_bounds__(64 * NW) void k_gqa_tiled_split(Params p)
{
    constexpr int SPAN = NW * NT * 64;                    // tokens a workgroup can cover
    constexpr int SC_BYTES = NW * NT * 4 * SROW * 4;      // scores [wave][block][head][SROW]
    constexpr int SCALE_BYTES = 2 * SPAN * 4;             // ks, vs of the span
    constexpr int RED_BYTES = NW * 4 * D * 4;             // [wave][head][d] fp32, reuses the space above
    constexpr int UNION = (SC_BYTES + SCALE_BYTES > RED_BYTES) ? SC_BYTES + SCALE_BYTES : RED_BYTES;
    static_assert(SPAN <= 4 * 64 * NW, "one float4 of each scale array per thread");
    __shared__ __attribute__((aligned(16))) char s_mem[UNION];
    __shared__ __attribute__((aligned(16))) int8_t s_q[NW][4][D];
    __shared__ __attribute__((aligned(16))) float s_out[4][D];
    __shared__ float s_sq[NW][4], s_m[NW][4], s_l[NW][4], s_vmax[NW];
    float *s_sc = reinterpret_cast<float *>(s_mem);
    float *s_ks = reinterpret_cast<float *>(s_mem + SC_BYTES);
    float *s_vs = s_ks + SPAN;
    float *s_red = reinterpret_cast<float *>(s_mem);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int split = blockIdx.x, bkv = blockIdx.y;
    const int b = bkv / p.Hkv, kvh = bkv % p.Hkv;
    const int G = p.G;
    const int64_t pbase = (int64_t)bkv * gridDim.x + split;

    int T = p.T;
    if (p.seq_len) T = min(max(__builtin_amdgcn_readfirstlane(p.seq_len[b]), 0), p.T);
    const int blk_lo = split * p.blocks_per_split;
    const int t_lo = blk_lo * 64;
    if (t_lo >= T) {
        if constexpr (DIRECT) {
            // a sequence of length 0: a row of zeros
            for (int o = tid; o < G * D; o += 64 * NW) p.o[((int64_t)b * p.Hq + kvh * G) * D + o] = 0.0f;
        } else {
            // this split lies past the end of the sequence: an empty partial (weight 0 in the merge)
            for (int o = tid; o < 4 * D; o += 64 * NW) p.part_o[pbase * 4 * D + o] = 0.0f;
            if (tid < 4) {
                p.part_ml[pbase * 8 + tid] = -INFINITY;
                p.part_ml[pbase * 8 + 4 + tid] = 0.0f;
            }
        }
        return;
    }
    const int t_end = min((blk_lo + p.blocks_per_split) * 64, T);   // first token this workgroup does not own
    const int nblk_row = p.Tstride >> 6;                            // blocks per cache row

    // ---- loads, in the order they are needed: the span's scales, the query rows, then the ring
    const int sidx = 4 * tid;   // one float4 of each scale array per thread
    float4 ks4 = make_float4(0.f, 0.f, 0.f, 0.f), vs4 = ks4;
    const int last_blk = (T - 1) >> 6;   // the last block that holds a token of this sequence
    if (sidx < SPAN) {
        if (p.block_table) {
            // four consecutive tokens lie in one page; blocks past the sequence's last one (their table entries may
            // hold anything) fall back on it, and their tokens are masked like any token past the end
            const int tb = min((t_lo + sidx) >> 6, last_blk);
            const int64_t page = p.block_table[(int64_t)b * p.max_pages + tb];
            const int64_t at = (page * p.Hkv + kvh) * 64 + ((t_lo + sidx) & 63);
            ks4 = *reinterpret_cast<const float4 *>(p.ks + at);
            vs4 = *reinterpret_cast<const float4 *>(p.vs + at);
        } else {
            const int tk = min(t_lo + sidx, p.Tstride - 4);   // the row's own memory; tokens past the end are masked
            ks4 = *reinterpret_cast<const float4 *>(p.ks + (int64_t)bkv * p.Tstride + tk);
            vs4 = *reinterpret_cast<const float4 *>(p.vs + (int64_t)bkv * p.Tstride + tk);
        }
    }
    const int hr = lane >> 4, jj = lane & 15;
    const int head = kvh * G + min(hr, G - 1);
    const float *qr = p.q + ((int64_t)b * p.Hq + head) * D;
    const float4 qlo = *reinterpret_cast<const float4 *>(qr + 4 * jj);
    const float4 qhi = *reinterpret_cast<const float4 *>(qr + 64 + 4 * jj);

    // block j of this wave: index blk_lo + NW*j + wave (the waves stream neighbouring blocks); blocks past the
    // end of the cache row fall back on its last block and are masked like any token past the end
    const int r16 = lane & 15, c4 = lane >> 4;
    // (both layouts put lane l's 16 bytes at 16*l inside each 1 KB piece: uniform base + one per-lane offset)
    const unsigned loff = 16u * (unsigned)lane;
    const int8_t *kblk[NT], *vblk[NT];   // the wave's blocks: 8 KB each, at the same offset in both arrays
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        int64_t off;
        if (p.block_table) {   // one scalar table look-up per block
            const int page = __builtin_amdgcn_readfirstlane(
                p.block_table[(int64_t)b * p.max_pages + min(blk_lo + NW * j + wave, last_blk)]);
            off = ((int64_t)page * p.Hkv + kvh) * 8192;
        } else {
            off = ((int64_t)bkv * nblk_row + min(blk_lo + NW * j + wave, nblk_row - 1)) * 8192;
        }
        kblk[j] = p.kq + off;
        vblk[j] = p.vt + off;
    }

    // load unit u in [0, 16 * NT): units 0 .. 8*NT-1 are key loads (block u/8; 16 tokens u%8/2, d half u%2),
    // the rest value loads (block (u - 8*NT)/8; head-dim rows 16*(u%8) .. +15); unit u lives in slot u % RING
    v4i ring[RING];
    auto issue = [&](auto U) {
        constexpr int u = decltype(U)::value;
        if constexpr (u < 8 * NT) {
            constexpr int j = u / 8, sub = (u % 8) / 2, hf = u % 2;
            ring[u % RING] = *reinterpret_cast<const v4i *>(kblk[j] + (sub * 2048 + hf * 1024) + loff);
        } else if constexpr (u < 16 * NT) {
            constexpr int j = (u - 8 * NT) / 8, n = u % 8;
            ring[u % RING] = *reinterpret_cast<const v4i *>(vblk[j] + n * 1024 + loff);
        }
    };
    __builtin_amdgcn_sched_barrier(0);
    static_for<RING>([&](auto U) { issue(U); });
    __builtin_amdgcn_sched_barrier(0);

    // ---- scales of the span -> LDS, and the largest V scale among the live tokens
    {
        const float v[4] = {vs4.x, vs4.y, vs4.z, vs4.w};
        float vm = 0.0f;
#pragma unroll
        for (int e = 0; e < 4; ++e) vm = fmaxf(vm, (t_lo + sidx + e < t_end) ? v[e] : 0.0f);
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) vm = fmaxf(vm, __shfl_xor(vm, off, 64));
        if (sidx < SPAN) {
            *reinterpret_cast<float4 *>(s_ks + sidx) = ks4;
            *reinterpret_cast<float4 *>(s_vs + sidx) = vs4;
        }
        if (lane == 0) s_vmax[wave] = vm;
    }
    // ---- query heads of this group: every wave rotates and quantizes them for itself
    {
        float v[8] = {qlo.x, qlo.y, qlo.z, qlo.w, qhi.x, qhi.y, qhi.z, qhi.w};
        fwht_chunk<D>(v, jj);
        float a = abs8(v);
        a = fmax_xor<1>(a); a = fmax_xor<2>(a); a = fmax_xor<4>(a); a = fmax_xor<8>(a);
        const float sc = (a == 0.0f) ? 1.0f : a / 127.0f;
        const float inv = (a == 0.0f) ? 0.0f : 127.0f / a;
        const uint32_t c0 = quant4(v[0], v[1], v[2], v[3], inv), c1 = quant4(v[4], v[5], v[6], v[7], inv);
        *reinterpret_cast<uint32_t *>(&s_q[wave][hr][4 * jj]) = c0;
        *reinterpret_cast<uint32_t *>(&s_q[wave][hr][64 + 4 * jj]) = c1;
        if (jj == 0) s_sq[wave][hr] = sc;
        if (p.dbg_qq && split == 0 && wave == 0 && hr < G) {
            int8_t *dq = p.dbg_qq + ((int64_t)b * p.Hq + head) * D;
            *reinterpret_cast<uint32_t *>(dq + 4 * jj) = c0;
            *reinterpret_cast<uint32_t *>(dq + 64 + 4 * jj) = c1;
            if (jj == 0) p.dbg_sq[(int64_t)b * p.Hq + head] = sc;
        }
    }
    // LDS only: the ring's loads stay in flight across this barrier
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    float vmax = s_vmax[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) vmax = fmaxf(vmax, s_vmax[w]);
    const float fix = vmax > 0.0f ? FIX_ONE / vmax : 0.0f;   // weight -> fixed point
    // MFMA operand B of the score product: column l%16 = query head (columns >= G are zero), 16-byte chunk l/16
    v4i qb0 = {0, 0, 0, 0}, qb1 = {0, 0, 0, 0};
    if (r16 < G) {
        qb0 = *reinterpret_cast<const v4i *>(&s_q[wave][r16][16 * c4]);
        qb1 = *reinterpret_cast<const v4i *>(&s_q[wave][r16][64 + 16 * c4]);
    }
    const float cq = r16 < G ? s_sq[wave][r16] * p.score_scale : 0.0f;   // this lane's head, log2 units

    // ---- pass 1: scores.  Lane (head r16, group c4) gets tokens 16*sub + 4*c4 .. +3 of each 16-token product.
    float *sc_wave = s_sc + wave * (NT * 4 * SROW);
    float mrun = -INFINITY;
    static_for<NT>([&](auto J) {
        constexpr int j = decltype(J)::value;
        const int tok0 = (blk_lo + NW * j + wave) * 64;        // first token of the block (may lie past t_end)
        const int sbase = (NW * j + wave) * 64;                // its place in the staged scales
        static_for<4>([&](auto S) {
            constexpr int sub = decltype(S)::value;
            constexpr int u = 8 * j + 2 * sub;
            v4i dots = __builtin_amdgcn_mfma_i32_16x16x64_i8(ring[u % RING], qb0, (v4i){0, 0, 0, 0}, 0, 0, 0);
            dots = __builtin_amdgcn_mfma_i32_16x16x64_i8(ring[(u + 1) % RING], qb1, dots, 0, 0, 0);
            issue(std::integral_constant<int, u + RING>{});
            issue(std::integral_constant<int, u + 1 + RING>{});
            __builtin_amdgcn_sched_barrier(0);
            const float4 kk = *reinterpret_cast<const float4 *>(s_ks + sbase + 16 * sub + 4 * c4);
            const int tt = tok0 + 16 * sub + 4 * c4;
            if (p.dbg_dots && r16 < G) {
                int32_t *dd = p.dbg_dots + ((int64_t)b * p.Hq + kvh * G + r16) * p.T;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (tt + e < t_end) dd[tt + e] = dots[e];
            }
            float4 sc;
            sc.x = (float)dots[0] * (kk.x * cq);
            sc.y = (float)dots[1] * (kk.y * cq);
            sc.z = (float)dots[2] * (kk.z * cq);
            sc.w = (float)dots[3] * (kk.w * cq);
            if (tok0 + 64 > t_end) {   // the block holds the end of the span (uniform over the wave)
                sc.x = (tt + 0 < t_end) ? sc.x : -INFINITY;
                sc.y = (tt + 1 < t_end) ? sc.y : -INFINITY;
                sc.z = (tt + 2 < t_end) ? sc.z : -INFINITY;
                sc.w = (tt + 3 < t_end) ? sc.w : -INFINITY;
            }
            if (r16 < 4) *reinterpret_cast<float4 *>(sc_wave + (j * 4 + r16) * SROW + 16 * sub + 4 * c4) = sc;
            mrun = fmaxf(fmaxf(mrun, fmaxf(sc.x, sc.y)), fmaxf(sc.z, sc.w));
        });
    });
    // maximum per head over the wave's tokens: lanes r16, r16 + 16, r16 + 32, r16 + 48 hold the partial maxima
    mrun = fmaxf(mrun, xor_lane<16>(mrun));
    mrun = fmaxf(mrun, __shfl_xor(mrun, 32, 64));
    if (lane < 4) s_m[wave][lane] = mrun;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // ---- pass 2: P.V.  Row r16 = 4*head + digit of operand A.  The four lanes of a quad share a head: lane `dg`
    // of the quad computes the weights of tokens 16*c4 + 4*dg .. +3 of the block (one exp2 per weight and lane, not
    // four), as 28-bit fixed-point codes; every lane then takes its own 7-bit digit of all 16 codes of the quad
    // (quad broadcasts).  The softmax is taken against the wave's own maximum (a wave whose tokens are all masked
    // has maximum -inf: its weights are 0, and 0 stands in for the maximum).
    const int hh = r16 >> 2, dg = r16 & 3;
    const float m_raw = s_m[wave][hh];
    const float m_h = (m_raw == -INFINITY) ? 0.0f : m_raw;
    const unsigned sh = 21u - 7u * (unsigned)dg;
    v4i acc[8];
#pragma unroll
    for (int n = 0; n < 8; ++n) acc[n] = (v4i){0, 0, 0, 0};
    float lsum = 0.0f;
    static_for<NT>([&](auto J) {
        constexpr int j = decltype(J)::value;
        const float4 s4 = *reinterpret_cast<const float4 *>(sc_wave + (j * 4 + hh) * SROW + 16 * c4 + 4 * dg);
        const float4 v4 = *reinterpret_cast<const float4 *>(s_vs + (NW * j + wave) * 64 + 16 * c4 + 4 * dg);
        const float ss[4] = {s4.x, s4.y, s4.z, s4.w}, vv[4] = {v4.x, v4.y, v4.z, v4.w};
        unsigned code[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float pe = __builtin_amdgcn_exp2f(ss[e] - m_h);       // masked token: exp2(-inf) = 0
            lsum += pe;
            const float a = (pe == 0.0f) ? 0.0f : pe * (vv[e] * fix);   // (a masked token's scale may be anything)
            code[e] = min((unsigned)(a + 0.5f), 0x0fffffffu);           // to nearest; the clamp covers a = 2^28
        }
        v4i pa;
        static_for<4>([&](auto K) {
            constexpr int k = decltype(K)::value;   // tokens 16*c4 + 4*k .. +3: the codes of quad lane k
            unsigned word = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const unsigned c = (unsigned)__builtin_amdgcn_update_dpp(0, (int)code[e], k * 0x55, 0xf, 0xf, true);
                word |= ((c >> sh) & 0x7fu) << (8 * e);
            }
            pa[k] = (int)word;
        });
        static_for<8>([&](auto N) {
            constexpr int n = decltype(N)::value;
            constexpr int u = 8 * NT + 8 * j + n;
            acc[n] = __builtin_amdgcn_mfma_i32_16x16x64_i8(pa, ring[u % RING], acc[n], 0, 0, 0);
            issue(std::integral_constant<int, u + RING>{});
        });
    });
    // the sum of the weights of head hh: over the quad, then over the four chunks c4
    lsum += xor_lane<1>(lsum);
    lsum += xor_lane<2>(lsum);
    lsum += xor_lane<16>(lsum);
    lsum += __shfl_xor(lsum, 32, 64);
    if ((lane & 0x33) == 0) s_l[wave][hh] = lsum;   // lanes 0, 4, 8, 12

    // ---- digits -> fp32.  Lane (r16, c4) holds column d = 16*n + r16 of rows 4*c4 + i: digit i of head c4, worth
    // 2^(21 - 7*i) / fix: the four digits of a value are the four registers of one lane (low digits added first).
    float val[8];
    {
        const float unit = vmax > 0.0f ? vmax / FIX_ONE : 0.0f;
#pragma unroll
        for (int n = 0; n < 8; ++n) {
            float f = (float)acc[n][3] * unit;
            f += (float)acc[n][2] * (unit * 128.0f);
            f += (float)acc[n][1] * (unit * 16384.0f);
            f += (float)acc[n][0] * (unit * 2097152.0f);
            val[n] = f;
        }
    }
    // ---- the waves meet.  Every wave is done with the scores and scales before their space is reused.
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    {
        float *dst = s_red + (wave * 4 + c4) * D + r16;
#pragma unroll
        for (int n = 0; n < 8; ++n) dst[16 * n] = val[n];
    }
    __syncthreads();
    // rescale each wave's sums from its own maximum to the common one; thread -> (d, two heads)
    if (tid < 256) {
        const int d = tid & (D - 1), hp = (tid >> 7) * 2;
        float m2[2] = {s_m[0][hp], s_m[0][hp + 1]};
#pragma unroll
        for (int w = 1; w < NW; ++w) {
            m2[0] = fmaxf(m2[0], s_m[w][hp]);
            m2[1] = fmaxf(m2[1], s_m[w][hp + 1]);
        }
        float sum[2] = {0.0f, 0.0f}, l[2] = {0.0f, 0.0f};
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float2 v = make_float2(s_red[(w * 4 + hp) * D + d], s_red[(w * 4 + hp + 1) * D + d]);
            const float f0 = (s_m[w][hp] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(s_m[w][hp] - m2[0]);
            const float f1 = (s_m[w][hp + 1] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(s_m[w][hp + 1] - m2[1]);
            sum[0] += v.x * f0;
            sum[1] += v.y * f1;
            l[0] += s_l[w][hp] * f0;
            l[1] += s_l[w][hp + 1] * f1;
        }
        if constexpr (DIRECT) {
            s_out[hp][d] = l[0] > 0.0f ? sum[0] * (1.0f / l[0]) : 0.0f;
            s_out[hp + 1][d] = l[1] > 0.0f ? sum[1] * (1.0f / l[1]) : 0.0f;
        } else {
            p.part_o[(pbase * 4 + hp) * D + d] = sum[0];
            p.part_o[(pbase * 4 + hp + 1) * D + d] = sum[1];
            if (d == 0) {
                p.part_ml[pbase * 8 + hp] = m2[0];
                p.part_ml[pbase * 8 + hp + 1] = m2[1];
                p.part_ml[pbase * 8 + 4 + hp] = l[0];
                p.part_ml[pbase * 8 + 4 + hp + 1] = l[1];
            }
        }
    }
    if constexpr (DIRECT) {
        __syncthreads();
        if (tid < 64 && hr < G) {   // 16 lanes per head row, as the merge kernel has them
            float v[8];
            const float4 lo = *reinterpret_cast<const float4 *>(&s_out[hr][4 * jj]);
            const float4 hi = *reinterpret_cast<const float4 *>(&s_out[hr][64 + 4 * jj]);
            v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w;
            v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
            if (!p.out_rotated) fwht_chunk<D>(v, jj);
            float *orow = p.o + ((int64_t)b * p.Hq + kvh * G + hr) * D;
            *reinterpret_cast<float4 *>(orow + 4 * jj) = make_float4(v[0], v[1], v[2], v[3]);
            *reinterpret_cast<float4 *>(orow + 64 + 4 * jj) = make_float4(v[4], v[5], v[6], v[7]);
        }
    }
}

// Row-major codes [rows, src_stride tokens, 128] -> the two tiled layouts, one workgroup per (64-token block, row,
// which): keys into 16-token tiles [8 chunks][16 tokens][16 bytes] (a straight permutation of 16-byte pieces),
// values into transposed blocks through LDS (tokens >= T inside the last block touched: 0).
__global__ __launch_bounds__(256) void k_tiled_from_rows(const int8_t *__restrict__ kq, const int8_t *__restrict__ vq,
                                                         int8_t *__restrict__ kt, int8_t *__restrict__ vt, int T,
                                                         int64_t src_stride, int64_t dst_stride, int z0)
{
    __shared__ __attribute__((aligned(16))) int8_t s[64][D + 16];
    const int tid = threadIdx.x, blk = blockIdx.x;
    const int64_t row = blockIdx.y;
    const bool is_v = (int)blockIdx.z + z0 != 0;   // z0 = 1: values only
    const int8_t *src = (is_v ? vq : kq) + (row * src_stride + (int64_t)blk * 64) * D;
    int8_t *dst = (is_v ? vt : kt) + (row * dst_stride + (int64_t)blk * 64) * D;
    if (!is_v) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + 256 * i, t = c >> 3, part = c & 7;   // 16-byte chunk `part` of token t
            v4i v = {0, 0, 0, 0};
            if (blk * 64 + t < T) v = *reinterpret_cast<const v4i *>(src + t * D + 16 * part);
            *reinterpret_cast<v4i *>(dst + (t >> 4) * 2048 + part * 256 + (t & 15) * 16) = v;
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int c = tid + 256 * i, t = c >> 3, part = c & 7;
        v4i v = {0, 0, 0, 0};
        if (blk * 64 + t < T) v = *reinterpret_cast<const v4i *>(src + t * D + 16 * part);
        *reinterpret_cast<v4i *>(&s[t][16 * part]) = v;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int c = tid + 256 * i, d = c >> 2, part = c & 3;   // tokens 16*part .. +15 of head-dim row d
        uint32_t w[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            uint32_t x = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) x |= (uint32_t)(uint8_t)s[16 * part + 4 * k + e][d] << (8 * e);
            w[k] = x;
        }
        *reinterpret_cast<uint4 *>(dst + (d >> 4) * 1024 + part * 256 + (d & 15) * 16) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

// The decode step's append for this layout: rotate + quantize the new token's key and value heads exactly as
// k_kv_append does (fwht_quant.hip); the key codes go to their 128-byte line, the value codes to byte t % 64 of
// the 128 head-dim rows of block t / 64.  16 lanes per head; blockIdx.y = 0: keys, 1: values.
// ROPE: rows are fused QKV rows [Hq | Hkv | Hkv] x 128 and query / key heads first get the rotary embedding
// (the arithmetic of k_rope_kv_append, layer_ops.hip); queries leave packed in q_out.
template <bool ROPE>
__global__ __launch_bounds__(256) void k_kv_append_vt(const float *__restrict__ k_new, const float *__restrict__ v_new,
                                                      int64_t row_stride, const float *__restrict__ cs,
                                                      const float *__restrict__ sn, float *__restrict__ q_out,
                                                      int8_t *__restrict__ kq, float *__restrict__ ks,
                                                      int8_t *__restrict__ vt, float *__restrict__ vs,
                                                      const int32_t *__restrict__ pos, int B, int Hq, int Hkv, int T_cap,
                                                      const int32_t *__restrict__ block_table, int max_pages)
{
    constexpr int LPB = 16;
    const int t = threadIdx.x, j = t % LPB;
    const int heads = ROPE ? Hq + 2 * Hkv : Hkv;
    const int flat = blockIdx.x * 16 + t / LPB;
    const int b = min(flat / heads, B - 1), hd = flat % heads;
    bool is_q = false, is_v;
    int h;
    const float *src;
    if constexpr (ROPE) {
        is_q = hd < Hq;
        is_v = hd >= Hq + Hkv;
        h = is_v ? hd - Hq - Hkv : hd - Hq;
        src = k_new + (int64_t)b * row_stride + (int64_t)hd * D + 4 * j;
    } else {
        is_v = blockIdx.y != 0;
        h = hd;
        src = (is_v ? v_new : k_new) + (int64_t)b * row_stride + (int64_t)h * D + 4 * j;
    }
    const int tp = pos[b];
    const bool live = flat < B * heads && tp >= 0 && tp < T_cap;
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
    if constexpr (ROPE) {
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
    }
    fwht_chunk<D>(v, j);   // every lane takes part in the cross-lane stages
    float a = abs8(v);
#pragma unroll
    for (int m = LPB / 2; m >= 1; m >>= 1) a = fmaxf(a, __shfl_xor(a, m, 64));
    const float sc = (a == 0.0f) ? 1.0f : a / 127.0f;
    const float inv = (a == 0.0f) ? 0.0f : 127.0f / a;
    if (live && !is_q) {
        // first token of the 64-token block that holds tp: in the sequence's own row, or in its page of the pool
        const int64_t blk0 = block_table ? ((int64_t)block_table[(int64_t)b * max_pages + (tp >> 6)] * Hkv + h) * 64
                                         : ((int64_t)b * Hkv + h) * T_cap + (tp & ~63);
        const uint32_t c0 = quant4(v[0], v[1], v[2], v[3], inv), c1 = quant4(v[4], v[5], v[6], v[7], inv);
        if (j == 0) (is_v ? vs : ks)[blk0 + (tp & 63)] = sc;
        if (!is_v) {
            // codes 4j .. 4j+3: chunk j/4, bytes 4*(j%4) .. of token tp % 16 in tile tp / 16; codes 64 + 4j ..: chunk 4 + j/4
            int8_t *q = kq + (blk0 + (tp & 48)) * D + (j >> 2) * 256 + (tp & 15) * 16 + 4 * (j & 3);
            *reinterpret_cast<uint32_t *>(q) = c0;
            *reinterpret_cast<uint32_t *>(q + 1024) = c1;
        } else {
            // code d of token tp: block tp / 64, piece d / 16, token chunk (tp % 64) / 16, row d % 16, byte tp % 16
            int8_t *blk = vt + blk0 * D + (j >> 2) * 1024 + ((tp & 63) >> 4) * 256 +
                          4 * (j & 3) * 16 + (tp & 15);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                blk[e * 16] = (int8_t)(c0 >> (8 * e));
                blk[4096 + e * 16] = (int8_t)(c1 >> (8 * e));
            }
        }
    }
}

constexpr int NT_MAX = 4;

struct Plan {
    int splits, per;   // workgroups per cache row, 64-token blocks per workgroup
};

// Blocks per workgroup: 16 (four per wave) when that still gives every compute unit a workgroup, otherwise as few as
// it takes to get there.
static Plan pick(int64_t B, int64_t Hkv, int64_t T)
{
    const int blocks = (int)((T + 63) / 64);
    const int64_t rows = B * Hkv, cus = compute_units();
    Plan pl;
    pl.per = 4 * NT_MAX;
    pl.splits = (blocks + pl.per - 1) / pl.per;
    if (rows * pl.splits < cus) {
        int want = (int)((cus + rows - 1) / rows);
        if (want > blocks) want = blocks;
        pl.per = (blocks + want - 1) / want;
        pl.splits = (blocks + pl.per - 1) / pl.per;
    }
    return pl;
}

// the largest split count pick() returns for any length in [1, T]
int max_splits(int64_t B, int64_t Hkv, int64_t T)
{
    const int blocks = (int)((T + 63) / 64);
    const int64_t rows = B * Hkv, cus = compute_units();
    int best = (blocks + 4 * NT_MAX - 1) / (4 * NT_MAX);
    int want = (int)((cus + rows - 1) / rows);
    if (want > blocks) want = blocks;
    if (rows < cus && want > best) best = want;
    return best;
}

}  // namespace avt
}  // namespace mi

using namespace mi;

static int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

struct ScoreGate {
    int8_t *qq;
    float *sq;
    int32_t *dots;
};

static int32_t run_tiled(const float *q, const int8_t *kq, const float *ks, const int8_t *vt, const float *vs, float *o,
                      int8_t *oq, float *oscale, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T_cap,
                      const int32_t *seq_len, int64_t T_max, int32_t out_rotated, void *workspace,
                      int64_t workspace_bytes, hipStream_t s, const int32_t *block_table = nullptr,
                      int64_t max_pages = 0, const ScoreGate *dbg = nullptr)
{
    if (block_table) {   // paged: the capacity of a sequence is its share of the table
        if (max_pages <= 0 || max_pages > (1 << 18) || !seq_len || !aligned4(block_table)) return MI_EINVAL;
        T_cap = max_pages * 64;
    }
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || T_cap <= 0 || T_max <= 0 || T_max > T_cap) return MI_EINVAL;
    if (D != avt::D || Hq % Hkv || Hq / Hkv > 4 || T_cap % 64) return MI_EINVAL;
    if (T_cap > (1LL << 24) || B * Hkv > 65535) return MI_ERANGE;
    if (!q || !kq || !ks || !vt || !vs || !workspace) return MI_EINVAL;
    if (!aligned16(q) || !aligned16(kq) || !aligned16(vt) || !aligned16(ks) || !aligned16(vs) || !aligned16(workspace))
        return MI_EINVAL;
    if (seq_len && !aligned4(seq_len)) return MI_EINVAL;
    if (workspace_bytes < mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T_max)) return MI_ENOSPC;
    const avt::Plan plan = avt::pick(B, Hkv, T_max);
    // one workgroup sees the whole sequence: it writes the output rows (the gate takes the split form: it wants no o)
    const bool direct = plan.splits == 1 && !oq && !dbg;
    avt::Params p;
    p.q = q; p.kq = kq; p.ks = ks; p.vt = vt; p.vs = vs;
    p.Hq = (int)Hq; p.Hkv = (int)Hkv; p.G = (int)(Hq / Hkv); p.T = (int)T_max;
    p.Tstride = (int)T_cap;
    p.seq_len = seq_len;
    p.score_scale = 1.4426950408889634f * 0.08838834764831845f;  // log2(e) / sqrt(128)
    p.o = o; p.out_rotated = out_rotated;
    p.block_table = block_table; p.max_pages = (int)max_pages;
    p.dbg_qq = dbg ? dbg->qq : nullptr;
    p.dbg_sq = dbg ? dbg->sq : nullptr;
    p.dbg_dots = dbg ? dbg->dots : nullptr;
    p.part_o = static_cast<float *>(workspace);
    p.part_ml = reinterpret_cast<float *>(static_cast<char *>(workspace) +
                                          align_up(B * Hkv * plan.splits * 4 * avt::D * 4, 256));
    p.blocks_per_split = plan.per;
    const dim3 grid((unsigned)plan.splits, (unsigned)(B * Hkv));
    const int nt = (plan.per + 3) / 4;
#define MI_TILED(NT_, DIR_) hipLaunchKernelGGL((avt::k_gqa_tiled_split<4, NT_, 8, DIR_>), grid, dim3(256), 0, s, p)
    if (direct) { if (nt <= 1) MI_TILED(1, true); else if (nt <= 2) MI_TILED(2, true); else MI_TILED(4, true); }
    else { if (nt <= 1) MI_TILED(1, false); else if (nt <= 2) MI_TILED(2, false); else MI_TILED(4, false); }
#undef MI_TILED
    if (direct || dbg) return launch_status();
    int32_t rc = launch_status();
    if (rc) return rc;
    return attn::launch_merge(p.part_o, p.part_ml, o, oq, oscale, B, Hq, Hkv, plan.splits, out_rotated, s);
}

extern "C" int32_t mi_gqa_decode_attn_tiled(const float *q, const int8_t *kq, const float *ks, const int8_t *vt,
                                         const float *vs, float *o, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                                         int64_t T_cap, const int32_t *seq_len, int64_t T_max, int32_t out_rotated,
                                         void *workspace, int64_t workspace_bytes, void *stream)
{
    if (!o || !aligned16(o)) return MI_EINVAL;
    return run_tiled(q, kq, ks, vt, vs, o, nullptr, nullptr, B, Hq, Hkv, D, T_cap, seq_len, T_max, out_rotated, workspace,
                  workspace_bytes, as_stream(stream));
}

extern "C" int32_t mi_gqa_decode_attn_tiled_quant_i8(const float *q, const int8_t *kq, const float *ks, const int8_t *vt,
                                                  const float *vs, float *o_rot, int8_t *oq, float *oscale, int64_t B,
                                                  int64_t Hq, int64_t Hkv, int64_t D, int64_t T_cap,
                                                  const int32_t *seq_len, int64_t T_max, void *workspace,
                                                  int64_t workspace_bytes, void *stream)
{
    if (!oq || !oscale || !aligned4(oq) || !aligned4(oscale) || (o_rot && !aligned16(o_rot))) return MI_EINVAL;
    if (Hq > 64) return MI_ERANGE;
    return run_tiled(q, kq, ks, vt, vs, o_rot, oq, oscale, B, Hq, Hkv, D, T_cap, seq_len, T_max, 1, workspace,
                  workspace_bytes, as_stream(stream));
}

// Gate helper for this layout: the split kernel alone, which also writes out the int8 query codes, their scales and
// the raw int32 dots it works from (no merge, no o).
extern "C" int32_t mi_gqa_decode_scores_tiled_i32(const float *q, const int8_t *kt, const float *ks, const int8_t *vt,
                                                  const float *vs, int8_t *qq, float *sq, int32_t *dots, int64_t B,
                                                  int64_t Hq, int64_t Hkv, int64_t D, int64_t T_cap, int64_t T,
                                                  void *workspace, int64_t workspace_bytes, void *stream)
{
    if (!qq || !sq || !dots || !aligned4(qq) || !aligned4(sq) || !aligned4(dots)) return MI_EINVAL;
    const ScoreGate g = {qq, sq, dots};
    return run_tiled(q, kt, ks, vt, vs, nullptr, nullptr, nullptr, B, Hq, Hkv, D, T_cap, nullptr, T, 1, workspace,
                     workspace_bytes, as_stream(stream), nullptr, 0, &g);
}

namespace mi {
int32_t launch_linear_fused(const float *, const int8_t *, const float *, float *, int8_t *, float *, int64_t, int64_t,
                            int64_t, hipStream_t, bool);
}

// Attention and the output projection behind it as one call.  Workspace: the merged rows (fp32, rotated basis), their
// codes and their scales (offsets that depend on B and Hq alone), then the attention's own.
extern "C" int64_t mi_gqa_decode_attn_linear_workspace_bytes(int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T)
{
    const int64_t a = mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T);
    if (a < 0) return a;
    return a + align_up(B * Hq * D * 4, 256) + align_up(B * Hq * D, 256) + align_up(B * 4, 256);
}

extern "C" int32_t mi_gqa_decode_attn_tiled_linear_f32(const float *q, const int8_t *kq, const float *ks,
                                                       const int8_t *vt, const float *vs, float *o_rot,
                                                       const int8_t *qw, const float *sw, float *y, int64_t B,
                                                       int64_t Hq, int64_t Hkv, int64_t D, int64_t T_cap,
                                                       const int32_t *seq_len, int64_t T_max, int64_t N,
                                                       void *workspace, int64_t workspace_bytes, void *stream)
{
    if (!qw || !sw || !y || !workspace || N <= 0 || N % 16) return MI_EINVAL;
    if (!aligned16(qw) || !aligned16(sw) || !aligned16(y) || !aligned16(workspace) || (o_rot && !aligned16(o_rot)))
        return MI_EINVAL;
    if (Hq > 64) return MI_ERANGE;
    const int64_t attn_bytes = mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T_max);
    if (attn_bytes < 0) return (int32_t)attn_bytes;
    if (workspace_bytes < mi_gqa_decode_attn_linear_workspace_bytes(B, Hq, Hkv, D, T_max)) return MI_ENOSPC;
    const int64_t K = Hq * D;
    char *base = static_cast<char *>(workspace);
    float *row = reinterpret_cast<float *>(base);
    int8_t *oq = reinterpret_cast<int8_t *>(base + align_up(B * K * 4, 256));
    float *oscale = reinterpret_cast<float *>(reinterpret_cast<char *>(oq) + align_up(B * K, 256));
    void *attn_ws = reinterpret_cast<char *>(oscale) + align_up(B * 4, 256);
    hipStream_t s = as_stream(stream);
    if (B == 1 && (K == 2048 || K == 4096)) {
        // One token: merging its Hq rows AND quantizing them in one workgroup makes that workgroup read every split's
        // partials (Hq x splits x 512 B, half a megabyte at 32 splits) through one compute unit.  Here the merge runs
        // over many workgroups and leaves the fp32 row; the projection's GEMV quantizes it in its own prologue
        // (the same row quantizer on the same values: identical codes, scale and y).
        float *orow = o_rot ? o_rot : row;
        int32_t rc = run_tiled(q, kq, ks, vt, vs, orow, nullptr, nullptr, B, Hq, Hkv, D, T_cap, seq_len, T_max, 1, attn_ws,
                               attn_bytes, s);
        if (rc) return rc;
        return launch_linear_fused(orow, qw, sw, y, oq, oscale, 1, N, K, s, false);
    }
    int32_t rc = run_tiled(q, kq, ks, vt, vs, o_rot, oq, oscale, B, Hq, Hkv, D, T_cap, seq_len, T_max, 1, attn_ws,
                           attn_bytes, s);
    if (rc) return rc;
    return mi_w8a8_gemm_dequant_f32(oq, oscale, qw, sw, y, B, N, K, stream);
}

extern "C" int32_t mi_kv_tiled_from_rows_i8(const int8_t *kq, const int8_t *vq, int8_t *kt, int8_t *vt, int64_t rows,
                                            int64_t T, int64_t src_stride, int64_t T_cap, void *stream)
{
    if ((!kq && !vq) || (kq && !kt) || (vq && !vt)) return MI_EINVAL;
    if (rows <= 0 || T <= 0 || T > src_stride || T > T_cap || T_cap % 64) return MI_EINVAL;
    if ((kq && (!aligned16(kq) || !aligned16(kt))) || (vq && (!aligned16(vq) || !aligned16(vt)))) return MI_EINVAL;
    if (rows > 65535 || T_cap > (1LL << 24)) return MI_ERANGE;
    const unsigned blocks = (unsigned)((T + 63) / 64);
    const dim3 grid(blocks, (unsigned)rows, (kq && vq) ? 2 : 1);
    hipLaunchKernelGGL(avt::k_tiled_from_rows, grid, dim3(256), 0, as_stream(stream), kq, vq, kt, vt, (int)T, src_stride,
                       T_cap, (kq ? 0 : 1));
    return launch_status();
}

static int32_t check_append(const void *a, const void *b, const void *kq, const void *ks, const void *vt,
                            const void *vs, const void *pos, int64_t B, int64_t Hkv, int64_t D, int64_t T_cap)
{
    if (!a || !b || !kq || !ks || !vt || !vs || !pos) return MI_EINVAL;
    if (B <= 0 || Hkv <= 0 || T_cap <= 0 || T_cap % 64 || D != 128) return MI_EINVAL;
    if (B * Hkv > (1LL << 24) || T_cap > (1LL << 24)) return MI_ERANGE;
    if (!aligned16(a) || !aligned16(b) || !aligned4(kq) || !aligned4(ks) || !aligned4(vs) || !aligned4(pos))
        return MI_EINVAL;
    return MI_OK;
}

extern "C" int32_t mi_kv_append_tiled_f32_i8(const float *k_new, const float *v_new, int64_t row_stride, int8_t *kq,
                                          float *ks, int8_t *vt, float *vs, const int32_t *pos, int64_t B,
                                          int64_t Hkv, int64_t D, int64_t T_cap, void *stream)
{
    int32_t rc = check_append(k_new, v_new, kq, ks, vt, vs, pos, B, Hkv, D, T_cap);
    if (rc) return rc;
    if (row_stride < Hkv * D || row_stride % 4) return MI_EINVAL;
    const dim3 grid((unsigned)((B * Hkv + 15) / 16), 2);
    hipLaunchKernelGGL(avt::k_kv_append_vt<false>, grid, dim3(256), 0, as_stream(stream), k_new, v_new, row_stride,
                       (const float *)nullptr, (const float *)nullptr, (float *)nullptr, kq, ks, vt, vs, pos, (int)B, 0,
                       (int)Hkv, (int)T_cap, (const int32_t *)nullptr, 0);
    return launch_status();
}

extern "C" int32_t mi_rope_kv_append_tiled_f32_i8(const float *qkv, int64_t row_stride, const float *rope_cos,
                                               const float *rope_sin, float *q_out, int8_t *kq, float *ks,
                                               int8_t *vt, float *vs, const int32_t *pos, int64_t B, int64_t Hq,
                                               int64_t Hkv, int64_t D, int64_t T_cap, void *stream)
{
    int32_t rc = check_append(qkv, q_out, kq, ks, vt, vs, pos, B, Hkv, D, T_cap);
    if (rc) return rc;
    if (!rope_cos || !rope_sin || !aligned16(rope_cos) || !aligned16(rope_sin) || Hq <= 0) return MI_EINVAL;
    if (row_stride < (Hq + 2 * Hkv) * D || row_stride % 4) return MI_EINVAL;
    const int64_t heads = B * (Hq + 2 * Hkv);
    hipLaunchKernelGGL(avt::k_kv_append_vt<true>, dim3((unsigned)((heads + 15) / 16)), dim3(256), 0, as_stream(stream),
                       qkv, (const float *)nullptr, row_stride, rope_cos, rope_sin, q_out, kq, ks, vt, vs, pos, (int)B,
                       (int)Hq, (int)Hkv, (int)T_cap, (const int32_t *)nullptr, 0);
    return launch_status();
}

// ---- the paged form of the tiled cache: pools of 64-token pages, one page = one 8 KB key block (four 16-token tiles)
// and one 8 KB transposed value block per kv head, so the attention kernel's loads stay 1 KB contiguous and a block
// costs it one scalar table look-up.
extern "C" int32_t mi_gqa_decode_attn_tiled_paged(const float *q, const int8_t *kt_pool, const float *ks_pool,
                                                  const int8_t *vt_pool, const float *vs_pool, float *o,
                                                  const int32_t *block_table, int64_t max_pages, int64_t B,
                                                  int64_t Hq, int64_t Hkv, int64_t D, const int32_t *seq_len,
                                                  int64_t T_max, int32_t out_rotated, void *workspace,
                                                  int64_t workspace_bytes, void *stream)
{
    if (!o || !aligned16(o) || !block_table) return MI_EINVAL;
    return run_tiled(q, kt_pool, ks_pool, vt_pool, vs_pool, o, nullptr, nullptr, B, Hq, Hkv, D, 0, seq_len, T_max,
                     out_rotated, workspace, workspace_bytes, as_stream(stream), block_table, max_pages);
}

extern "C" int32_t mi_gqa_decode_attn_tiled_paged_quant_i8(const float *q, const int8_t *kt_pool, const float *ks_pool,
                                                           const int8_t *vt_pool, const float *vs_pool, float *o_rot,
                                                           int8_t *oq, float *oscale, const int32_t *block_table,
                                                           int64_t max_pages, int64_t B, int64_t Hq, int64_t Hkv,
                                                           int64_t D, const int32_t *seq_len, int64_t T_max,
                                                           void *workspace, int64_t workspace_bytes, void *stream)
{
    if (!oq || !oscale || !aligned4(oq) || !aligned4(oscale) || (o_rot && !aligned16(o_rot)) || !block_table) return MI_EINVAL;
    if (Hq > 64) return MI_ERANGE;
    return run_tiled(q, kt_pool, ks_pool, vt_pool, vs_pool, o_rot, oq, oscale, B, Hq, Hkv, D, 0, seq_len, T_max, 1,
                     workspace, workspace_bytes, as_stream(stream), block_table, max_pages);
}

extern "C" int32_t mi_kv_append_tiled_paged_f32_i8(const float *k_new, const float *v_new, int64_t row_stride,
                                                   int8_t *kt_pool, float *ks_pool, int8_t *vt_pool, float *vs_pool,
                                                   const int32_t *block_table, int64_t max_pages, const int32_t *pos,
                                                   int64_t B, int64_t Hkv, int64_t D, void *stream)
{
    if (!block_table || !aligned4(block_table) || max_pages <= 0 || max_pages > (1 << 18)) return MI_EINVAL;
    int32_t rc = check_append(k_new, v_new, kt_pool, ks_pool, vt_pool, vs_pool, pos, B, Hkv, D, max_pages * 64);
    if (rc) return rc;
    if (row_stride < Hkv * D || row_stride % 4) return MI_EINVAL;
    const dim3 grid((unsigned)((B * Hkv + 15) / 16), 2);
    hipLaunchKernelGGL(avt::k_kv_append_vt<false>, grid, dim3(256), 0, as_stream(stream), k_new, v_new, row_stride,
                       (const float *)nullptr, (const float *)nullptr, (float *)nullptr, kt_pool, ks_pool, vt_pool,
                       vs_pool, pos, (int)B, 0, (int)Hkv, (int)(max_pages * 64), block_table, (int)max_pages);
    return launch_status();
}

extern "C" int32_t mi_rope_kv_append_tiled_paged_f32_i8(const float *qkv, int64_t row_stride, const float *rope_cos,
                                                        const float *rope_sin, float *q_out, int8_t *kt_pool,
                                                        float *ks_pool, int8_t *vt_pool, float *vs_pool,
                                                        const int32_t *block_table, int64_t max_pages,
                                                        const int32_t *pos, int64_t B, int64_t Hq, int64_t Hkv,
                                                        int64_t D, void *stream)
{
    if (!block_table || !aligned4(block_table) || max_pages <= 0 || max_pages > (1 << 18)) return MI_EINVAL;
    int32_t rc = check_append(qkv, q_out, kt_pool, ks_pool, vt_pool, vs_pool, pos, B, Hkv, D, max_pages * 64);
    if (rc) return rc;
    if (!rope_cos || !rope_sin || !aligned16(rope_cos) || !aligned16(rope_sin) || Hq <= 0) return MI_EINVAL;
    if (row_stride < (Hq + 2 * Hkv) * D || row_stride % 4) return MI_EINVAL;
    const int64_t heads = B * (Hq + 2 * Hkv);
    hipLaunchKernelGGL(avt::k_kv_append_vt<true>, dim3((unsigned)((heads + 15) / 16)), dim3(256), 0, as_stream(stream),
                       qkv, (const float *)nullptr, row_stride, rope_cos, rope_sin, q_out, kt_pool, ks_pool, vt_pool,
                       vs_pool, pos, (int)B, (int)Hq, (int)Hkv, (int)(max_pages * 64), block_table, (int)max_pages);
    return launch_status();
}
