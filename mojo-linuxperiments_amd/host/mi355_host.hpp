// C++ host layer over the C ABI (include/mi355_int8.h).
//
// The upstream library is Mojo and its host types are move-only RAII structs
// that report failure through `__bool__`, null pointers and Bool returns
// (threading/numa_arena.mojo:6, :32-38, :46-52; threading/linux_threading.mojo:43,
// :70-80, :103-121).  No Mojo toolchain exists where this is built, so the same
// surface is written in C++: DeviceArena mirrors NumaArena, StreamPool mirrors
// ThreadPool, Gate mirrors MutexGate, and QuantLinear / DecodeAttention /
// KvCache / DecoderLayer / DecoderStack / MoeFfn are the quantize / linear / attention / MoE call surface that a Mojo
// host would hold as structs over the same handles.  Nothing here throws.
#pragma once
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <utility>

#include "../../include/mi355_int8.h"

namespace mi355 {

class Context {
public:
    explicit Context(int device = 0) { if (mi_ctx_create(device, &h_) != MI_OK) h_ = nullptr; }
    ~Context() { if (h_) mi_ctx_destroy(h_); }
    Context(Context &&o) noexcept : h_(o.h_) { o.h_ = nullptr; }
    Context(const Context &) = delete;
    Context &operator=(const Context &) = delete;
    explicit operator bool() const { return h_ != nullptr; }
    mi_ctx *handle() const { return h_; }
    int compute_units() const { return h_ ? mi_ctx_compute_units(h_) : 0; }

private:
    mi_ctx *h_ = nullptr;
};

// NumaArena[alignment] -> DeviceArena<Alignment> (numa_arena.mojo:5-87)
template <int64_t Alignment = 256>
class DeviceArena {
public:
    DeviceArena(const Context &ctx, int64_t size) : size_(size)
    {
        if (!ctx || mi_arena_create(ctx.handle(), size, Alignment, &h_) != MI_OK) { h_ = nullptr; size_ = 0; }
    }
    ~DeviceArena() { if (h_) mi_arena_destroy(h_); }
    DeviceArena(DeviceArena &&o) noexcept : h_(o.h_), size_(o.size_) { o.h_ = nullptr; o.size_ = 0; }
    DeviceArena(const DeviceArena &) = delete;
    DeviceArena &operator=(const DeviceArena &) = delete;
    explicit operator bool() const { return h_ != nullptr; }

    // Pointer to uninitialized device memory, or nullptr if the arena is exhausted.
    template <typename T>
    T *alloc(int64_t count = 1) { return h_ ? static_cast<T *>(mi_arena_alloc(h_, count * (int64_t)sizeof(T))) : nullptr; }
    int64_t mark() const { return h_ ? mi_arena_mark(h_) : 0; }
    void reset_to(int64_t watermark) { if (h_) (void)mi_arena_reset_to(h_, watermark); }
    void reset() { if (h_) (void)mi_arena_reset(h_); }
    int64_t remaining() const { return h_ ? mi_arena_remaining(h_) : 0; }
    int64_t used() const { return h_ ? mi_arena_used(h_) : 0; }
    bool verify_placement() const { return !h_ || mi_arena_verify_placement(h_) == 1; }

private:
    mi_arena *h_ = nullptr;
    int64_t size_ = 0;
};

// Pinned host staging slab on one NUMA node: NumaArena as it is (numa_arena.mojo:5-87), with pages the
// device can copy from at link rate.
template <int64_t Alignment = 256>
class HostArena {
public:
    HostArena(const Context &ctx, int node, int64_t size) : node_(node)
    {
        if (!ctx || mi_host_arena_create(ctx.handle(), size, Alignment, node, &h_) != MI_OK) h_ = nullptr;
    }
    ~HostArena() { if (h_) mi_arena_destroy(h_); }
    HostArena(HostArena &&o) noexcept : h_(o.h_), node_(o.node_) { o.h_ = nullptr; }
    HostArena(const HostArena &) = delete;
    HostArena &operator=(const HostArena &) = delete;
    explicit operator bool() const { return h_ != nullptr; }

    template <typename T>
    T *alloc(int64_t count = 1) { return h_ ? static_cast<T *>(mi_arena_alloc(h_, count * (int64_t)sizeof(T))) : nullptr; }
    int64_t mark() const { return h_ ? mi_arena_mark(h_) : 0; }
    void reset_to(int64_t watermark) { if (h_) (void)mi_arena_reset_to(h_, watermark); }
    void reset() { if (h_) (void)mi_arena_reset(h_); }
    int64_t remaining() const { return h_ ? mi_arena_remaining(h_) : 0; }
    int64_t used() const { return h_ ? mi_arena_used(h_) : 0; }
    bool verify_placement() const { return !h_ || mi_arena_verify_placement(h_) == 1; }
    int node() const { return node_; }

private:
    mi_arena *h_ = nullptr;
    int node_ = -1;
};

// MutexGate (linux_threading.mojo:174-198): trivially copyable token over a handle.
struct Gate {
    mi_gate *h = nullptr;
    static Gate create(const Context &ctx) { Gate g; if (mi_gate_create(ctx.handle(), &g.h) != MI_OK) g.h = nullptr; return g; }
    void destroy() { if (h) mi_gate_destroy(h); h = nullptr; }
    bool release(void *stream) const { return mi_gate_release(h, stream) == MI_OK; }
    bool wait(void *stream) const { return mi_gate_wait(h, stream) == MI_OK; }
    bool wait_host() const { return mi_gate_wait_host(h) == MI_OK; }
    void reset() const { (void)mi_gate_reset(h); }
};

// ThreadPool (linux_threading.mojo:43-158): launch / wait_all / wait_any over streams.
class StreamPool {
public:
    StreamPool(const Context &ctx, int capacity)
    {
        if (!ctx || mi_stream_pool_create(ctx.handle(), capacity, &h_) != MI_OK) h_ = nullptr;
    }
    ~StreamPool()
    {
        if (!h_) return;
        if (mi_stream_pool_destroy(h_) == MI_EBUSY) {
            // linux_threading.mojo:70-77: destroying a pool with live work is fatal
            std::fputs("FATAL: StreamPool destroyed with work in flight\n", stderr);
            std::abort();
        }
    }
    StreamPool(StreamPool &&o) noexcept : h_(o.h_) { o.h_ = nullptr; }
    StreamPool(const StreamPool &) = delete;
    StreamPool &operator=(const StreamPool &) = delete;
    explicit operator bool() const { return h_ != nullptr; }
    int size() const { return h_ ? mi_stream_pool_capacity(h_) : 0; }

    // func(stream, args...) is enqueued on the first free slot; false when the
    // pool is full or func reports a status other than MI_OK.  Never blocks.
    template <typename F, typename... Args>
    bool launch(F &&func, Args &&...args)
    {
        if (!h_) return false;
        const int32_t slot = mi_stream_pool_begin(h_);
        if (slot < 0) return false;
        const int32_t rc = func(mi_stream_pool_stream(h_, slot), std::forward<Args>(args)...);
        return mi_stream_pool_end(h_, slot) == MI_OK && rc == MI_OK;
    }
    void wait_all() { if (h_) (void)mi_stream_pool_wait_all(h_); }
    int wait_any() { return h_ ? mi_stream_pool_wait_any(h_) : -1; }
    void *stream(int slot) const { return h_ ? mi_stream_pool_stream(h_, slot) : nullptr; }

private:
    mi_stream_pool *h_ = nullptr;
};

// A Hadamard-rotated W8A8 linear layer with weights prepared once on the device.
template <int Block = 128>
struct QuantLinear {
    int8_t *qw = nullptr;
    float *sw = nullptr;
    void *workspace = nullptr;
    int64_t workspace_bytes = 0;
    int64_t N = 0, K = 0, max_tokens = 0;

    // w_dev: fp32 [N,K] in device memory.  false if the arena is exhausted.
    template <typename Arena>
    bool prepare(Arena &arena, const float *w_dev, int64_t n, int64_t k, int64_t max_m, void *stream)
    {
        N = n; K = k; max_tokens = max_m;
        qw = arena.template alloc<int8_t>(n * k);
        sw = arena.template alloc<float>(n);
        workspace_bytes = mi_w8a8_linear_workspace_bytes(max_m, n, k);
        workspace = workspace_bytes > 0 ? arena.template alloc<uint8_t>(workspace_bytes) : nullptr;
        if (!qw || !sw || !workspace) return false;
        return mi_fwht_quant_f32_i8(w_dev, qw, sw, n, k, Block, stream) == MI_OK;
    }
    // x fp32 [M,K] -> y fp32 [M,N]; status as in the C ABI
    int32_t forward(const float *x, float *y, int64_t M, void *stream) const
    {
        if (M > max_tokens) return MI_ERANGE;
        return mi_w8a8_linear_f32(x, qw, sw, y, M, N, K, Block, workspace, workspace_bytes, stream);
    }
};

// Several W8A8 contractions in one launch (mi_gemm_batch_*): made once for a list of shapes, run with the operands of
// each call.  Move-only; the tile lists live in arena memory.
struct GemmBatch {
    mi_gemm_batch *h = nullptr;
    void *plan = nullptr;
    int32_t n = 0;

    GemmBatch() = default;
    GemmBatch(const GemmBatch &) = delete;
    GemmBatch &operator=(const GemmBatch &) = delete;
    GemmBatch(GemmBatch &&o) noexcept : h(o.h), plan(o.plan), n(o.n) { o.h = nullptr; }
    ~GemmBatch() { if (h) mi_gemm_batch_destroy(h); }
    explicit operator bool() const { return h != nullptr; }

    // mnk: [count][3] = M, N, K per problem.  Status as in the C ABI (MI_ENOMEM: the arena is exhausted).
    template <typename Arena>
    int32_t prepare(Arena &arena, const int64_t *mnk, int32_t count)
    {
        const int64_t bytes = mi_gemm_batch_plan_bytes(mnk, count);
        if (bytes < 0) return (int32_t)bytes;
        plan = arena.template alloc<uint8_t>(bytes);
        if (!plan) return MI_ENOMEM;
        n = count;
        return mi_gemm_batch_create(mnk, count, plan, bytes, &h);
    }
    int32_t run(const mi_gemm_problem *problems, void *stream) const { return mi_gemm_batch_run_f32(h, problems, stream); }
    int32_t run_i32(const mi_gemm_problem *problems, void *stream) const { return mi_gemm_batch_run_i32(h, problems, stream); }
};

// Decode attention over an int8 KV cache held by the caller.
struct DecodeAttention {
    int64_t B = 0, Hq = 0, Hkv = 0, D = 128, T = 0;
    void *workspace = nullptr;
    int64_t workspace_bytes = 0;

    template <typename Arena>
    bool prepare(Arena &arena, int64_t b, int64_t hq, int64_t hkv, int64_t t)
    {
        B = b; Hq = hq; Hkv = hkv; T = t;
        workspace_bytes = mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T);
        if (workspace_bytes <= 0) return false;
        workspace = arena.template alloc<uint8_t>(workspace_bytes);
        return workspace != nullptr;
    }
    // appends nothing: quantizes `rows` fp32 rows [rows,128] into cache codes + scales
    static int32_t quantize_rows(const float *kv, int8_t *codes, float *scales, int64_t rows, void *stream)
    {
        return mi_fwht_quant_f32_i8(kv, codes, scales, rows, 128, 128, stream);
    }
    int32_t forward(const float *q, const int8_t *kq, const float *ks, const int8_t *vq, const float *vs, float *o,
                    bool out_rotated, void *stream) const
    {
        return mi_gqa_decode_attn(q, kq, ks, vq, vs, o, B, Hq, Hkv, D, T, out_rotated ? 1 : 0, workspace,
                                  workspace_bytes, stream);
    }
};

// An int8 KV cache of fixed capacity held in an arena: the decode loop appends one token per sequence at its own
// position and attends over what each sequence holds.  Positions and lengths are int32 [B] arrays in device memory
// (the loop that produces them runs on the device side of the stream, not on the host).
// tiled: the codes live in the layouts the int8 matrix instruction loads straight from memory (keys in 16-token
// tiles, values in transposed 64-token blocks; capacity a multiple of 64 tokens): the fast attention path.
// Otherwise both halves are row-major [B, Hkv, T_cap, 128].  Same arithmetic, same codes, same scales.  The layout is
// the caller's choice at prepare() and never follows from the capacity; code that fills kq / vq itself must write
// the layout it chose (load_rows() converts row-major codes).
struct KvCache {
    int64_t B = 0, Hq = 0, Hkv = 0, D = 128, T_cap = 0;
    bool tiled = false;
    int8_t *kq = nullptr, *vq = nullptr;
    float *ks = nullptr, *vs = nullptr;
    void *workspace = nullptr;
    int64_t workspace_bytes = 0;

    template <typename Arena>
    bool prepare(Arena &arena, int64_t b, int64_t hq, int64_t hkv, int64_t t_cap, bool use_tiled_layouts)
    {
        B = b; Hq = hq; Hkv = hkv; T_cap = t_cap; tiled = use_tiled_layouts;
        if (tiled && T_cap % 64) return false;
        // sized for attend_project: the largest of the attend calls' workspaces
        workspace_bytes = mi_gqa_decode_attn_linear_workspace_bytes(B, Hq, Hkv, D, T_cap);
        if (workspace_bytes <= 0) return false;
        kq = arena.template alloc<int8_t>(B * Hkv * T_cap * D);
        vq = arena.template alloc<int8_t>(B * Hkv * T_cap * D);
        ks = arena.template alloc<float>(B * Hkv * T_cap);
        vs = arena.template alloc<float>(B * Hkv * T_cap);
        workspace = arena.template alloc<uint8_t>(workspace_bytes);
        return kq && vq && ks && vs && workspace;
    }
    explicit operator bool() const { return workspace != nullptr; }
    // k_new / v_new: head h of sequence b at + b*row_stride + h*128 floats (slices of a fused QKV row are fine)
    int32_t append(const float *k_new, const float *v_new, int64_t row_stride, const int32_t *pos, void *stream) const
    {
        return tiled ? mi_kv_append_tiled_f32_i8(k_new, v_new, row_stride, kq, ks, vq, vs, pos, B, Hkv, D, T_cap, stream)
                     : mi_kv_append_f32_i8(k_new, v_new, row_stride, kq, ks, vq, vs, pos, B, Hkv, D, T_cap, stream);
    }
    // a fused QKV row per sequence: rotary embedding on query and key heads, queries out, keys and values appended
    int32_t rope_append(const float *qkv, int64_t row_stride, const float *rope_cos, const float *rope_sin, float *q_out,
                        const int32_t *pos, void *stream) const
    {
        return tiled ? mi_rope_kv_append_tiled_f32_i8(qkv, row_stride, rope_cos, rope_sin, q_out, kq, ks, vq, vs, pos, B, Hq,
                                                      Hkv, D, T_cap, stream)
                     : mi_rope_kv_append_f32_i8(qkv, row_stride, rope_cos, rope_sin, q_out, kq, ks, vq, vs, pos, B, Hq, Hkv, D,
                                                T_cap, stream);
    }
    // t_max bounds every entry of seq_len (<= T_cap); the workspace serves every t_max up to the capacity
    int32_t attend(const float *q, float *o, const int32_t *seq_len, int64_t t_max, bool out_rotated, void *stream) const
    {
        return tiled ? mi_gqa_decode_attn_tiled(q, kq, ks, vq, vs, o, B, Hq, Hkv, D, T_cap, seq_len, t_max,
                                                out_rotated ? 1 : 0, workspace, workspace_bytes, stream)
                     : mi_gqa_decode_attn_cache(q, kq, ks, vq, vs, o, B, Hq, Hkv, D, T_cap, seq_len, t_max,
                                                out_rotated ? 1 : 0, workspace, workspace_bytes, stream);
    }
    // the same with the merge fused with the output projection's row quantizer (rows stay in the rotated basis of V)
    int32_t attend_quant(const float *q, float *o_rot, int8_t *oq, float *oscale, const int32_t *seq_len, int64_t t_max,
                         void *stream) const
    {
        return tiled ? mi_gqa_decode_attn_tiled_quant_i8(q, kq, ks, vq, vs, o_rot, oq, oscale, B, Hq, Hkv, D, T_cap, seq_len,
                                                         t_max, workspace, workspace_bytes, stream)
                     : mi_gqa_decode_attn_cache_quant_i8(q, kq, ks, vq, vs, o_rot, oq, oscale, B, Hq, Hkv, D, T_cap, seq_len,
                                                         t_max, workspace, workspace_bytes, stream);
    }
    // attention and the output projection behind it (prepared weights qw [N, Hq*128], sw [N]) as one call: y fp32 [B, N].
    // Tiled layouts only; o_rot (optional) receives the merged rows.
    int32_t attend_project(const float *q, float *o_rot, const int8_t *qw, const float *sw, float *y, int64_t N,
                           const int32_t *seq_len, int64_t t_max, void *stream) const
    {
        if (!tiled) return MI_EINVAL;
        return mi_gqa_decode_attn_tiled_linear_f32(q, kq, ks, vq, vs, o_rot, qw, sw, y, B, Hq, Hkv, D, T_cap, seq_len, t_max,
                                                   N, workspace, workspace_bytes, stream);
    }
    // a cache quantized in one go (prefill): row-major codes [B*Hkv, T, 128] (rows src_stride tokens apart) into this
    // cache's layout, first T tokens of every row; the scales are the caller's to copy into ks / vs
    int32_t load_rows(const int8_t *kq_rows, const int8_t *vq_rows, int64_t T, int64_t src_stride, void *stream) const
    {
        if (tiled) return mi_kv_tiled_from_rows_i8(kq_rows, vq_rows, kq, vq, B * Hkv, T, src_stride, T_cap, stream);
        if (src_stride != T_cap) return MI_EINVAL;
        int32_t rc = mi_memcpy_d2d(kq, kq_rows, B * Hkv * T_cap * D, stream);
        return rc == MI_OK ? mi_memcpy_d2d(vq, vq_rows, B * Hkv * T_cap * D, stream) : rc;
    }
};

// The same cache as pools of pages shared by all sequences: tokens [i*P, (i+1)*P) of sequence b live in page
// table[b*max_pages + i].  The table is the caller's (int32 in device memory): a scheduler hands pages out.
// tiled (pages of 64 tokens only): a page holds, per kv head, one 8 KB block of key tiles and one 8 KB transposed
// value block, the layouts of the tiled KvCache, so attention runs the matrix-instruction kernel at the dense
// layout's speed; otherwise pages are row-major [page_size, 128] per kv head.
struct PagedKvCache {
    int64_t B = 0, Hq = 0, Hkv = 0, D = 128, pages = 0, page_size = 0, max_pages = 0;
    bool tiled = false;
    int8_t *kq = nullptr, *vq = nullptr;
    float *ks = nullptr, *vs = nullptr;
    void *workspace = nullptr;
    int64_t workspace_bytes = 0;

    template <typename Arena>
    bool prepare(Arena &arena, int64_t b, int64_t hq, int64_t hkv, int64_t n_pages, int64_t p_size, int64_t max_pages_per_seq,
                 bool use_tiled_layouts)
    {
        B = b; Hq = hq; Hkv = hkv; pages = n_pages; page_size = p_size; max_pages = max_pages_per_seq;
        tiled = use_tiled_layouts;
        if (tiled && page_size != 64) return false;
        workspace_bytes = mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, max_pages * page_size);
        if (workspace_bytes <= 0) return false;
        kq = arena.template alloc<int8_t>(pages * Hkv * page_size * D);
        vq = arena.template alloc<int8_t>(pages * Hkv * page_size * D);
        ks = arena.template alloc<float>(pages * Hkv * page_size);
        vs = arena.template alloc<float>(pages * Hkv * page_size);
        workspace = arena.template alloc<uint8_t>(workspace_bytes);
        return kq && vq && ks && vs && workspace;
    }
    explicit operator bool() const { return workspace != nullptr; }
    int32_t append(const float *k_new, const float *v_new, int64_t row_stride, const int32_t *table, const int32_t *pos,
                   void *stream) const
    {
        return tiled ? mi_kv_append_tiled_paged_f32_i8(k_new, v_new, row_stride, kq, ks, vq, vs, table, max_pages, pos, B,
                                                       Hkv, D, stream)
                     : mi_kv_append_paged_f32_i8(k_new, v_new, row_stride, kq, ks, vq, vs, table, max_pages, page_size, pos,
                                                 B, Hkv, D, stream);
    }
    // a fused QKV row per sequence: rotary embedding, queries out, keys and values appended (tiled pages only)
    int32_t rope_append(const float *qkv, int64_t row_stride, const float *rope_cos, const float *rope_sin, float *q_out,
                        const int32_t *table, const int32_t *pos, void *stream) const
    {
        if (!tiled) return MI_EINVAL;
        return mi_rope_kv_append_tiled_paged_f32_i8(qkv, row_stride, rope_cos, rope_sin, q_out, kq, ks, vq, vs, table,
                                                    max_pages, pos, B, Hq, Hkv, D, stream);
    }
    int32_t attend(const float *q, float *o, const int32_t *table, const int32_t *seq_len, int64_t t_max, bool out_rotated,
                   void *stream) const
    {
        return tiled ? mi_gqa_decode_attn_tiled_paged(q, kq, ks, vq, vs, o, table, max_pages, B, Hq, Hkv, D, seq_len, t_max,
                                                      out_rotated ? 1 : 0, workspace, workspace_bytes, stream)
                     : mi_gqa_decode_attn_paged(q, kq, ks, vq, vs, o, table, max_pages, page_size, B, Hq, Hkv, D, seq_len,
                                                t_max, out_rotated ? 1 : 0, workspace, workspace_bytes, stream);
    }
    // the merge fused with the output projection's row quantizer (tiled pages only)
    int32_t attend_quant(const float *q, float *o_rot, int8_t *oq, float *oscale, const int32_t *table, const int32_t *seq_len,
                         int64_t t_max, void *stream) const
    {
        if (!tiled) return MI_EINVAL;
        return mi_gqa_decode_attn_tiled_paged_quant_i8(q, kq, ks, vq, vs, o_rot, oq, oscale, table, max_pages, B, Hq, Hkv, D,
                                                       seq_len, t_max, workspace, workspace_bytes, stream);
    }
};

// Router + top-k dispatch + grouped expert SwiGLU FFN.
struct MoeFfn {
    int64_t T = 0, H = 0, I = 0, E = 0;
    int32_t topk = 0;
    const float *wr = nullptr;
    const int8_t *wg = nullptr, *wu = nullptr, *wd = nullptr;
    const float *sg = nullptr, *su = nullptr, *sd = nullptr;
    void *workspace = nullptr;
    int64_t workspace_bytes = 0;

    template <typename Arena>
    bool prepare(Arena &arena, int64_t t, int64_t h, int64_t i, int64_t e, int32_t k)
    {
        T = t; H = h; I = i; E = e; topk = k;
        workspace_bytes = mi_moe_layer_workspace_bytes(T, H, I, E, topk);
        if (workspace_bytes <= 0) return false;
        workspace = arena.template alloc<uint8_t>(workspace_bytes);
        return workspace != nullptr;
    }
    int32_t forward(const float *x, float *y, void *stream) const
    {
        return mi_moe_layer(x, wr, wg, sg, wu, su, wd, sd, y, T, H, I, E, topk, workspace, workspace_bytes, stream);
    }
};

// One decoder layer of a decode step (one new token per sequence), chained on one stream, ten launches (eight for a single sequence):
// (residual +) RMSNorm + quantize -> QKV GEMV -> rotary + cache append -> attention over the cache (split, merge +
// quantize: the output projection takes the rows in the rotated basis of V) -> O GEMV -> residual + RMSNorm +
// quantize -> gate|up GEMV -> SwiGLU + quantize -> down GEMV (-> residual).
// Holds its prepared weights, its KV cache and its scratch rows in the arena.
struct DecoderLayer {
    int64_t B = 0, H = 0, Hq = 0, Hkv = 0, I = 0, T_cap = 0;
    float eps = 1e-5f;
    QuantLinear<128> qkv, o, gate_up, down;
    KvCache cache;
    // the MoE FFN in place of the dense one (gate_up / down stay unprepared): set by use_moe()
    const MoeFfn *moe = nullptr;
    const float *g1 = nullptr, *g2 = nullptr, *rope_cos = nullptr, *rope_sin = nullptr;
    // fp32 rows: layer input when it is a sum (h0), projections, attention output, residual stream after
    // attention (h1), down output (dn); xn / att (rotated basis) / hn / act only when prepare() was asked to trace
    float *h0 = nullptr, *qkv_out = nullptr, *q = nullptr, *ao = nullptr, *h1 = nullptr, *gu = nullptr, *dn = nullptr,
          *xn = nullptr, *att = nullptr, *hn = nullptr, *act = nullptr;
    // codes of the attention rows [B,Hq*128] and of the activated rows [B,I] (those of the normalized rows sit in
    // the workspaces of the QKV and gate|up projections)
    int8_t *ca = nullptr, *ci = nullptr;
    float *sa = nullptr, *si = nullptr;

    // fp32 weights in device memory: wqkv [(Hq+2Hkv)*128, H], wo [H, Hq*128], wgu [2I, H] (gate rows, then up
    // rows), wd [H, I]; norm weights g1, g2 [H]; rotary tables [T_cap, 64].  false if the arena is exhausted.
    template <typename Arena>
    bool prepare(Arena &arena, int64_t b, int64_t h, int64_t hq, int64_t hkv, int64_t i, int64_t t_cap, bool tiled_cache,
                 const float *wqkv, const float *wo, const float *wgu, const float *wd, const float *norm1,
                 const float *norm2, const float *cos_table, const float *sin_table, float epsilon, void *stream,
                 bool trace = false)
    {
        B = b; H = h; Hq = hq; Hkv = hkv; I = i; T_cap = t_cap; eps = epsilon;
        g1 = norm1; g2 = norm2; rope_cos = cos_table; rope_sin = sin_table;
        const int64_t nqkv = (Hq + 2 * Hkv) * 128;
        // wgu == wd == nullptr: the FFN half will be an MoE (use_moe)
        bool ok = qkv.prepare(arena, wqkv, nqkv, H, B, stream) && o.prepare(arena, wo, H, Hq * 128, B, stream) &&
                  (!wgu || gate_up.prepare(arena, wgu, 2 * I, H, B, stream)) &&
                  (!wd || down.prepare(arena, wd, H, I, B, stream)) && cache.prepare(arena, B, Hq, Hkv, T_cap, tiled_cache);
        h0 = arena.template alloc<float>(B * H);
        qkv_out = arena.template alloc<float>(B * nqkv);
        q = arena.template alloc<float>(B * Hq * 128);
        ao = arena.template alloc<float>(B * H);
        h1 = arena.template alloc<float>(B * H);
        gu = arena.template alloc<float>(B * 2 * I);
        dn = arena.template alloc<float>(B * H);
        ca = arena.template alloc<int8_t>(B * Hq * 128);
        ci = arena.template alloc<int8_t>(B * I);
        sa = arena.template alloc<float>(B);
        si = arena.template alloc<float>(B);
        if (trace) {
            xn = arena.template alloc<float>(B * H);
            att = arena.template alloc<float>(B * Hq * 128);
            hn = arena.template alloc<float>(B * H);
            act = arena.template alloc<float>(B * I);
            ok = ok && xn && att && hn && act;
        }
        return ok && h0 && qkv_out && q && ao && h1 && gu && dn && ca && ci && sa && si;
    }
    // The FFN half becomes residual + RMSNorm -> router, dispatch, grouped expert FFN (ffn prepared for T = B tokens,
    // hidden H; it must outlive the layer).  false if the arena is exhausted or the shapes disagree.
    template <typename Arena>
    bool use_moe(Arena &arena, const MoeFfn &ffn)
    {
        if (ffn.T != B || ffn.H != H || !ffn.workspace) return false;
        if (!hn) hn = arena.template alloc<float>(B * H);
        if (!hn) return false;
        moe = &ffn;
        return true;
    }
    // x fp32 [B,H], plus residual fp32 [B,H] or nullptr: the layer input is their sum (left in h0).  pos, seq_len
    // int32 [B] in device memory (seq_len = pos + 1 in a plain decode step); t_max bounds seq_len.  out fp32 [B,H],
    // or nullptr: the closing residual add is left to the next layer (give it x = dn, residual = h1).
    // The first failing call's status is returned.
    int32_t step(const float *x, const float *residual, const int32_t *pos, const int32_t *seq_len, int64_t t_max,
                 float *out, void *stream) const
    {
        // norm + quantize + projection: one kernel for a single token, two launches otherwise
        int32_t rc = mi_rmsnorm_linear_f32(x, residual, g1, eps, residual ? h0 : nullptr, xn, qkv.qw, qkv.sw, qkv_out, B,
                                           qkv.N, H, 128, qkv.workspace, qkv.workspace_bytes, stream);
        const float *xin = residual ? h0 : x;
        if (rc == MI_OK) rc = cache.rope_append(qkv_out, (Hq + 2 * Hkv) * 128, rope_cos, rope_sin, q, pos, stream);
        if (cache.tiled) {
            if (rc == MI_OK) rc = cache.attend_project(q, att, o.qw, o.sw, ao, H, seq_len, t_max, stream);
        } else {
            if (rc == MI_OK) rc = cache.attend_quant(q, att, ca, sa, seq_len, t_max, stream);
            if (rc == MI_OK) rc = mi_w8a8_gemm_dequant_f32(ca, sa, o.qw, o.sw, ao, B, H, Hq * 128, stream);
        }
        if (moe) {
            if (rc == MI_OK) rc = mi_rmsnorm_f32(ao, xin, g2, eps, h1, hn, B, H, stream);
            if (rc == MI_OK) rc = moe->forward(hn, dn, stream);
        } else {
            if (rc == MI_OK)
                rc = mi_rmsnorm_linear_f32(ao, xin, g2, eps, h1, hn, gate_up.qw, gate_up.sw, gu, B, 2 * I, H, 128,
                                           gate_up.workspace, gate_up.workspace_bytes, stream);
            if (rc == MI_OK) rc = mi_swiglu_quant_f32_i8(gu, act, ci, si, B, I, 128, stream);
            if (rc == MI_OK) rc = mi_w8a8_gemm_dequant_f32(ci, si, down.qw, down.sw, dn, B, H, I, stream);
        }
        if (rc == MI_OK && out) rc = mi_add_f32(h1, dn, out, B * H, stream);
        return rc;
    }
};

// A recorded sequence of launches, replayed as one (mi_graph_*).  Record with
//   Graph g; g.begin(stream); ...enqueue on stream...; g.end(stream);   then   g.launch(stream)
// after one eager run of the same calls (the first call of a kernel sets its attributes).  Move-only.
class Graph {
public:
    Graph() = default;
    Graph(const Graph &) = delete;
    Graph &operator=(const Graph &) = delete;
    Graph(Graph &&o) noexcept : h_(o.h_) { o.h_ = nullptr; }
    ~Graph() { if (h_) mi_graph_destroy(h_); }
    explicit operator bool() const { return h_ != nullptr; }
    int32_t begin(void *stream) { return mi_graph_capture_begin(stream); }
    int32_t end(void *stream)
    {
        if (h_) { mi_graph_destroy(h_); h_ = nullptr; }
        return mi_graph_capture_end(stream, &h_);
    }
    int32_t launch(void *stream) const { return h_ ? mi_graph_launch(h_, stream) : MI_EINVAL; }

private:
    mi_graph *h_ = nullptr;
};

// A stack of decoder layers for one decode step: layer l+1 takes x = dn and residual = h1 of layer l, so that the
// closing residual add of a layer happens inside the first kernel of the next one; only the last layer writes `out`.
// Capacity is a compile-time parameter like the reference's pool sizes; nothing is allocated outside the arena.
template <int MaxLayers = 128>
struct DecoderStack {
    DecoderLayer layers[MaxLayers];
    int count = 0;

    // appends a layer (arguments as DecoderLayer::prepare); false when the stack or the arena is full
    template <typename Arena, typename... Args>
    bool add(Arena &arena, Args &&...args)
    {
        if (count >= MaxLayers) return false;
        if (!layers[count].prepare(arena, std::forward<Args>(args)...)) return false;
        ++count;
        return true;
    }
    // one new token per sequence through every layer; the first failing call's status is returned
    int32_t step(const float *x, const int32_t *pos, const int32_t *seq_len, int64_t t_max, float *out, void *stream) const
    {
        if (count <= 0 || !out) return MI_EINVAL;
        const float *xin = x, *res = nullptr;
        for (int l = 0; l < count; ++l) {
            const int32_t rc = layers[l].step(xin, res, pos, seq_len, t_max, l + 1 == count ? out : nullptr, stream);
            if (rc != MI_OK) return rc;
            xin = layers[l].dn;
            res = layers[l].h1;
        }
        return MI_OK;
    }
};

}  // namespace mi355
