/*
 * mi355_int8.h — C ABI of libmi355_int8.so: the int8 inference hot path
 * (block-Hadamard rotation + int8 quantizer, W8A8 GEMM / GEMV, GQA decode
 * attention over an int8 KV cache, MoE top-k dispatch + grouped expert GEMM)
 * as hand-written HIP kernels for gfx950 (MI355X), plus the two runtime
 * pieces that stand in, on this path only, for the upstream NUMA arena and
 * clone3 thread pool.
 *
 * Calling convention (what a Mojo `external_call` / `DLHandle` binding, a cgo
 * stub or ctypes needs): every argument is a pointer, an int64_t or an
 * int32_t — the "args are 8-byte trivials" rule of the upstream launch path
 * (threading/linux_threading.mojo:106-112).  Errors are return values, never
 * exceptions and never exit(): 0 on success, a negative errno-class code
 * otherwise, the convention of the upstream syscall shim
 * (threading/linux.mojo:229-230, :235-236); allocation failure is a null
 * pointer (threading/numa_arena.mojo:46-52).
 *
 * Upstream has NO int8 kernels and no FFI (README.md:4, :10-13), so the
 * kernel entry points below replace nothing upstream; each cites the
 * workload element it implements.  The arena and stream-pool entry points do
 * replace upstream code and cite it.
 *
 * All device pointers must come from one device; kernels are enqueued on the
 * `stream` argument (a hipStream_t passed as void*, NULL = the null stream)
 * and return without waiting.  Calls are thread-compatible: no hidden mutable
 * globals, but one context / pool / arena must not be used from two threads
 * at once (upstream issues every launch from one orchestrator thread,
 * test_linux_threading.mojo:112-115).
 */
#ifndef MI355_INT8_H
#define MI355_INT8_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI_API __attribute__((visibility("default")))

/* ---- status codes (negative errno class) -------------------------------- */
#define MI_OK        0
#define MI_EIO      (-5)   /* a HIP runtime call failed; see mi_last_hip_error */
#define MI_ENOMEM   (-12)  /* device or host allocation failed                 */
#define MI_EBUSY    (-16)  /* no free slot / destroy while work is in flight   */
#define MI_ENODEV   (-19)  /* no such device, or not a gfx950 device           */
#define MI_EINVAL   (-22)  /* null pointer, bad shape, bad alignment           */
#define MI_ENOSPC   (-28)  /* workspace too small                              */
#define MI_ERANGE   (-34)  /* a size is beyond what the kernels support        */

MI_API const char *mi_status_string(int32_t status);
MI_API int32_t mi_last_hip_error(void);        /* hipError_t of the last MI_EIO on this thread */
MI_API int32_t mi_abi_version(void);

/* ---- context ------------------------------------------------------------- */
typedef struct mi_ctx mi_ctx;
MI_API int32_t mi_ctx_create(int32_t device, mi_ctx **out);
MI_API int32_t mi_ctx_destroy(mi_ctx *ctx);
MI_API int32_t mi_ctx_device(const mi_ctx *ctx);
MI_API int32_t mi_ctx_compute_units(const mi_ctx *ctx);
MI_API int64_t mi_ctx_memory_bytes(const mi_ctx *ctx);
MI_API int32_t mi_ctx_arch_name(const mi_ctx *ctx, char *buf, int64_t buf_len);

/* ---- device arena --------------------------------------------------------
 * Replaces NumaArena (threading/numa_arena.mojo:5-87) on this path: one slab
 * of device memory, bump allocation with an alignment, watermarks, a null
 * pointer on exhaustion, no per-allocation free.  `alignment` is a power of
 * two (numa_arena.mojo:139-140); the slab is zero-filled at creation the way
 * fresh mmap pages are (upstream tests rely on it, test_linux_threading.mojo:431). */
typedef struct mi_arena mi_arena;
MI_API int32_t mi_arena_create(mi_ctx *ctx, int64_t size_bytes, int64_t alignment, mi_arena **out); /* numa_arena.mojo:20-30 */
MI_API int32_t mi_arena_destroy(mi_arena *a);                  /* numa_arena.mojo:32-34 */
MI_API void   *mi_arena_alloc(mi_arena *a, int64_t bytes);     /* numa_arena.mojo:40-55; NULL when exhausted */
MI_API int64_t mi_arena_mark(const mi_arena *a);               /* numa_arena.mojo:57-59 */
MI_API int32_t mi_arena_reset_to(mi_arena *a, int64_t mark);   /* numa_arena.mojo:61-66; ignored (MI_EINVAL) unless 0 <= mark <= used */
MI_API int32_t mi_arena_reset(mi_arena *a);                    /* numa_arena.mojo:68-70 */
MI_API int64_t mi_arena_remaining(const mi_arena *a);          /* numa_arena.mojo:72-74 */
MI_API int64_t mi_arena_used(const mi_arena *a);               /* numa_arena.mojo:76-78 */
MI_API int32_t mi_arena_verify_placement(const mi_arena *a);   /* numa_arena.mojo:80-87; 1 = slab lives on the context's device (host slab: pinned host memory, on its node where the kernel can tell) */
/* Pinned host staging slab bound to one NUMA node (numa_node = -1: no binding), the host-side half of the
 * same allocator: mmap_numa + mbind(MPOL_BIND) (numa_arena.mojo:93-107), here as a memory policy held while
 * the runtime allocates the pinned pages.  Every mi_arena_* call above works on it; copies from it to the
 * device run at the full rate of the link (mi_memcpy_h2d is asynchronous only from pinned memory). */
MI_API int32_t mi_host_arena_create(mi_ctx *ctx, int64_t size_bytes, int64_t alignment, int32_t numa_node, mi_arena **out);

/* ---- stream pool and gate ------------------------------------------------
 * Replaces ThreadPool (threading/linux_threading.mojo:43-158) on this path:
 * a fixed number of slots, each a hipStream plus a completion event.  A slot
 * is "in use" from mi_stream_pool_end until its event has completed, as a
 * thread slot is from clone3 until child_tid returns to 0
 * (linux_threading.mojo:273-275).
 *   launch(fn, args)  ==  slot = begin(); enqueue work on stream(slot); end(slot)
 * begin never blocks and reports a full pool as MI_EBUSY, as launch returns
 * False (linux_threading.mojo:103-121). */
typedef struct mi_stream_pool mi_stream_pool;
/* capacity <= 1024.  A process has four hardware queues on this part (HIP's default): the first three slots run
 * beside each other and beside the null stream; a fourth and later slot shares a queue with an earlier one and
 * its work waits behind that slot's. */
MI_API int32_t mi_stream_pool_create(mi_ctx *ctx, int32_t capacity, mi_stream_pool **out); /* linux_threading.mojo:56-66, :130-158 */
MI_API int32_t mi_stream_pool_destroy(mi_stream_pool *p);      /* linux_threading.mojo:70-77: MI_EBUSY (pool kept) instead of abort() when work is in flight */
MI_API int32_t mi_stream_pool_capacity(const mi_stream_pool *p);         /* linux_threading.mojo:85-86 */
MI_API int32_t mi_stream_pool_begin(mi_stream_pool *p);        /* first free slot index, or MI_EBUSY; linux_threading.mojo:104-105 */
MI_API void   *mi_stream_pool_stream(mi_stream_pool *p, int32_t slot);   /* hipStream_t of the slot, NULL if out of range */
MI_API int32_t mi_stream_pool_end(mi_stream_pool *p, int32_t slot);      /* record the completion event: slot is now in use */
MI_API int32_t mi_stream_pool_in_use(mi_stream_pool *p, int32_t slot);   /* 1 / 0; frees the slot when its event has completed */
MI_API int32_t mi_stream_pool_wait_all(mi_stream_pool *p);     /* linux_threading.mojo:123-126 */
MI_API int32_t mi_stream_pool_wait_any(mi_stream_pool *p);     /* linux_threading.mojo:128-129, :391-407: index of a slot that finished, -1 if none was in use */

/* Replaces MutexGate (linux_threading.mojo:174-198): a one-shot token.
 * release() records it on a stream; wait() makes later work on another stream
 * wait for it, wait_host() makes the calling thread wait; waiting on a gate
 * that was never released is MI_EINVAL instead of blocking forever. */
typedef struct mi_gate mi_gate;
MI_API int32_t mi_gate_create(mi_ctx *ctx, mi_gate **out);
MI_API int32_t mi_gate_destroy(mi_gate *g);
MI_API int32_t mi_gate_release(mi_gate *g, void *stream);      /* linux_threading.mojo:191-194 */
MI_API int32_t mi_gate_wait(mi_gate *g, void *stream);         /* linux_threading.mojo:186-189: later work on `stream` waits */
MI_API int32_t mi_gate_wait_host(mi_gate *g);                  /* the calling host thread waits */
MI_API int32_t mi_gate_reset(mi_gate *g);                      /* linux_threading.mojo:196-198 */

/* ---- graphs ------------------------------------------------------------------
 * Decode-time chains of small kernels are launch-bound; a caller records the
 * chain once on a pool stream and replays it.  Every kernel entry point of
 * this library may be called between begin and end (none of them allocates,
 * synchronizes or records a memset node); call each one once eagerly first so
 * that one-time kernel attributes are already set.  No upstream counterpart:
 * a thread pool has no launch cost to amortize. */
typedef struct mi_graph mi_graph;
MI_API int32_t mi_graph_capture_begin(void *stream);           /* stream must not be the null stream */
MI_API int32_t mi_graph_capture_end(void *stream, mi_graph **out);
MI_API int32_t mi_graph_launch(mi_graph *g, void *stream);
MI_API int32_t mi_graph_destroy(mi_graph *g);

/* ---- copies, host staging, events ----------------------------------------- */
MI_API int32_t mi_memcpy_h2d(void *dst_dev, const void *src_host, int64_t bytes, void *stream);
MI_API int32_t mi_memcpy_d2h(void *dst_host, const void *src_dev, int64_t bytes, void *stream);
MI_API int32_t mi_memcpy_d2d(void *dst_dev, const void *src_dev, int64_t bytes, void *stream);
MI_API int32_t mi_fill_u32(void *dst_dev, uint32_t value, int64_t count, void *stream); /* a fill kernel, safe under graph capture */
MI_API int32_t mi_stream_synchronize(void *stream);
MI_API void   *mi_host_alloc(int64_t bytes);                   /* pinned host memory, NULL on failure */
MI_API int32_t mi_host_free(void *p);
typedef struct mi_event mi_event;
MI_API int32_t mi_event_create(mi_event **out);
MI_API int32_t mi_event_destroy(mi_event *e);
MI_API int32_t mi_event_record(mi_event *e, void *stream);
MI_API int32_t mi_event_synchronize(mi_event *e);
MI_API int32_t mi_event_elapsed_ms(mi_event *start, mi_event *stop, float *ms);

/* ---- a1 + a2 / a3 / a7: block Hadamard rotation fused with the row quantizer
 * x fp32 [M,K] row-major -> q int8 [M,K], scale fp32 [M].
 * Each row is rotated in blocks of `block` (128 or 256) along K with the
 * normalized Sylvester Hadamard matrix, then quantized symmetrically with its
 * own absmax: scale = a/127, code = clamp(rne(x' * (127/a)), -127, 127); an
 * all-zero row gives scale 1 and codes 0.  The same call prepares activations
 * (per token), weights [N,K] (per output channel) and KV-cache rows
 * [B*Hkv*T, D] (per token-head, block = D).  K % block == 0, K <= 32768.
 * Codes and scales are bit-exact against the CPU restatement.
 * Rows are meant to be finite (the rotation spreads one non-finite input over its whole block).  What the
 * quantizer does with a non-finite rotated value is fixed all the same, by IEEE max / min semantics: a NaN takes no
 * part in the absmax and gets the code -127; a row holding +-Inf gets scale Inf, code 0 for its finite values and
 * -127 for the infinite ones. */
MI_API int32_t mi_fwht_quant_f32_i8(const float *x, int8_t *q, float *scale,
                                    int64_t M, int64_t K, int32_t block, void *stream);
/* The same for several row sets in ONE launch (n <= 8; the prefill step's prologues: one set per distinct linear
 * input): every set as mi_fwht_quant_f32_i8 would do it, bit for bit; sets with K < 2048 or no rows make the call
 * fall back to one launch per set.  Sets must not overlap.  No upstream counterpart. */
typedef struct mi_quant_rows {
    const float *x;   /* fp32 [M,K] */
    int8_t *q;        /* int8 [M,K] */
    float *scale;     /* fp32 [M]   */
    int64_t M, K;
} mi_quant_rows;
MI_API int32_t mi_fwht_quant_batch_f32_i8(const mi_quant_rows *sets, int32_t n, int32_t block, void *stream);
/* a1 alone: out fp32 [M,K] = rotated rows (out may alias x). */
MI_API int32_t mi_fwht_f32(const float *x, float *out, int64_t M, int64_t K,
                           int32_t block, void *stream);

/* ---- a4 / a5: W8A8 contraction, acc[m,n] = sum_k qx[m,k] * qw[n,k]
 * qx int8 [M,K], qw int8 [N,K] (both K-contiguous), acc int32 [M,N].
 * M <= 64 streams the weights once through a skinny MFMA kernel (decode
 * GEMV); larger M uses the LDS-tiled v_mfma_i32_16x16x64_i8 kernel (prefill).
 * K % 128 == 0, N % 16 == 0.  Exact integer arithmetic. */
MI_API int32_t mi_w8a8_gemm_i32(const int8_t *qx, const int8_t *qw, int32_t *acc,
                                int64_t M, int64_t N, int64_t K, void *stream);
/* a4/a5 + a6 fused: y[m,n] = ((float)acc * sx[m]) * sw[n], fp32 [M,N]. */
MI_API int32_t mi_w8a8_gemm_dequant_f32(const int8_t *qx, const float *sx,
                                        const int8_t *qw, const float *sw, float *y,
                                        int64_t M, int64_t N, int64_t K, void *stream);
/* a4 for several contractions at once: ONE launch whose workgroups (one per compute unit) walk a list of 256 x 256
 * output tiles drawn from every problem of the batch, so that no problem's tile count has to divide by the number
 * of compute units, and no launch gap or first memory round trip lies between the problems.  No upstream
 * counterpart.  A batch is made once for a list of shapes
 * (mnk int64 [n][3] = M, N, K per problem; n <= 8; M >= 256, N >= 256, N % 16 == 0, K % 128 == 0, K >= 384, 127 * 127 * K < 2^31): the tile lists
 * are computed on the host and copied (synchronously) into `plan`, device memory of the caller of at least
 * mi_gemm_batch_plan_bytes(mnk, n) bytes that must stay untouched while the batch lives.  A run takes the operands
 * of this call (shapes must equal the batch's) and is an ordinary asynchronous launch: it may be captured into a
 * graph.  Outputs of different problems must not overlap.  Results equal those of mi_w8a8_gemm_dequant_f32 /
 * mi_w8a8_gemm_i32 on each problem, bit for bit. */
typedef struct mi_gemm_problem {
    const int8_t *qx;   /* int8 [M,K] */
    const float *sx;    /* fp32 [M]   (unused by the int32 form) */
    const int8_t *qw;   /* int8 [N,K] */
    const float *sw;    /* fp32 [N]   (unused by the int32 form) */
    void *out;          /* fp32 [M,N] (run_f32) or int32 [M,N] (run_i32), 16-byte aligned */
    int64_t M, N, K;
} mi_gemm_problem;
typedef struct mi_gemm_batch mi_gemm_batch;
MI_API int64_t mi_gemm_batch_plan_bytes(const int64_t *mnk, int32_t n);
/* The tile lists a batch would hold on a device of `compute_units` units, written to host memory (int32
 * [compute_units][per_wg][4] = problem or -1 for the end of a workgroup's list, first row, first column, cost in K
 * stages; workgroup w runs on XCD w % 8): for tests and for callers that want to look at the balance.  Returns the
 * bytes written.  Makes no device call. */
MI_API int64_t mi_gemm_batch_plan_host(const int64_t *mnk, int32_t n, int32_t compute_units, int32_t *lists_out,
                                       int64_t capacity_bytes, int32_t *per_wg_out);
MI_API int32_t mi_gemm_batch_create(const int64_t *mnk, int32_t n, void *plan, int64_t plan_bytes, mi_gemm_batch **out);
MI_API int32_t mi_gemm_batch_destroy(mi_gemm_batch *b);
MI_API int32_t mi_gemm_batch_run_f32(mi_gemm_batch *b, const mi_gemm_problem *problems, void *stream);
MI_API int32_t mi_gemm_batch_run_i32(mi_gemm_batch *b, const mi_gemm_problem *problems, void *stream);
/* a6 alone. */
MI_API int32_t mi_dequant_i32_f32(const int32_t *acc, const float *sx, const float *sw,
                                  float *y, int64_t M, int64_t N, void *stream);
/* The whole rotated W8A8 linear: x fp32 [M,K] -> y fp32 [M,N] with prepared
 * weights (qw, sw).  workspace holds the activation codes and scales. */
MI_API int64_t mi_w8a8_linear_workspace_bytes(int64_t M, int64_t N, int64_t K);
MI_API int32_t mi_w8a8_linear_f32(const float *x, const int8_t *qw, const float *sw, float *y,
                                  int64_t M, int64_t N, int64_t K, int32_t block,
                                  void *workspace, int64_t workspace_bytes, void *stream);
/* The same linear without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart upstream.  The activation
 * codes and scales live in a static device array of 8 MiB + 32 KiB that every device the library runs on holds
 * until the process ends; mi_ctx_create looks its address up for the context's device (otherwise the first call on
 * a device does).  Limits: M <= mi_w8a8_linear_noalloc_max_rows() = 8192 and M * K <=
 * mi_w8a8_linear_noalloc_max_codes() = 8 Mi, beyond them MI_ERANGE.  The call allocates and frees nothing.  All
 * calls on one device share the one array: two calls may not overlap on a device (different streams, or two
 * threads) - they would race on the codes; calls on one stream are ordered and safe.  Results are bit-identical to
 * mi_w8a8_linear_f32 (the same kernels run). */
MI_API int32_t mi_w8a8_linear_f32_noalloc(const float *x, const int8_t *qw, const float *sw, float *y,
                                          int64_t M, int64_t N, int64_t K, int32_t block, void *stream);
MI_API int64_t mi_w8a8_linear_noalloc_max_rows(void);
MI_API int64_t mi_w8a8_linear_noalloc_max_codes(void);

/* ---- a8: grouped-query decode attention over an int8 KV cache
 * q fp32 [B,Hq,D] (unrotated); kq,vq int8 [B,Hkv,T,D]; ks,vs fp32 [B,Hkv,T];
 * o fp32 [B,Hq,D].  D == 128, Hq % Hkv == 0, Hq/Hkv <= 4, any T >= 1.
 * The query head is rotated and quantized to int8, scores are int32 dots,
 * softmax (scale 1/sqrt(D)) and the P.V sum accumulate in fp32.
 * out_rotated != 0 leaves o in the rotated basis of V. */
MI_API int64_t mi_gqa_decode_workspace_bytes(int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T);
MI_API int32_t mi_gqa_decode_attn(const float *q, const int8_t *kq, const float *ks,
                                  const int8_t *vq, const float *vs, float *o,
                                  int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T,
                                  int32_t out_rotated, void *workspace, int64_t workspace_bytes,
                                  void *stream);
/* The same attention over a cache that is being filled: rows of kq/vq/ks/vs are T_cap tokens apart, sequence b
 * holds seq_len[b] tokens (int32 [B] in device memory; values outside [0, T_max] are clamped, a length of 0 gives
 * a row of zeros), T_max <= T_cap bounds every length and sizes the workspace
 * (mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T_max)).  No upstream counterpart: the step that follows
 * mi_kv_append_f32_i8 in a decode loop. */
MI_API int32_t mi_gqa_decode_attn_cache(const float *q, const int8_t *kq, const float *ks,
                                        const int8_t *vq, const float *vs, float *o,
                                        int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T_cap,
                                        const int32_t *seq_len, int64_t T_max, int32_t out_rotated,
                                        void *workspace, int64_t workspace_bytes, void *stream);
/* The same, with the merge of the splits fused with the int8 row quantizer of the output projection: per token the
 * Hq*D attention outputs are left in the rotated basis of V (block D) and quantized as one row, oq int8 [B,Hq*D] and
 * oscale fp32 [B], ready for mi_w8a8_gemm_dequant_f32 against output-projection weights that were prepared with
 * block D along K (x.H . (W.H)^T = x . W^T): neither the inverse rotation nor the projection's own rotation is
 * spent.  o_rot (optional, fp32 [B,Hq,D]) receives the row that was quantized.  Hq <= 64. */
MI_API int32_t mi_gqa_decode_attn_cache_quant_i8(const float *q, const int8_t *kq, const float *ks,
                                                 const int8_t *vq, const float *vs, float *o_rot,
                                                 int8_t *oq, float *oscale,
                                                 int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T_cap,
                                                 const int32_t *seq_len, int64_t T_max,
                                                 void *workspace, int64_t workspace_bytes, void *stream);
/* Paged layout of the same cache: the pools kq/vq int8 [pages, Hkv, P, D] and ks/vs fp32 [pages, Hkv, P] hold
 * pages of P = page_size tokens (a power of two, >= 16); tokens [i*P, (i+1)*P) of sequence b live in page
 * block_table[b*max_pages + i] (int32 in device memory; every entry that covers a token below seq_len[b], resp.
 * the position being appended, must be a valid page of the pool: the kernels cannot check it).  Same arithmetic
 * and same results as the dense layout.  No upstream counterpart. */
MI_API int32_t mi_gqa_decode_attn_paged(const float *q, const int8_t *kq_pool, const float *ks_pool,
                                        const int8_t *vq_pool, const float *vs_pool, float *o,
                                        const int32_t *block_table, int64_t max_pages, int64_t page_size,
                                        int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                                        const int32_t *seq_len, int64_t T_max, int32_t out_rotated,
                                        void *workspace, int64_t workspace_bytes, void *stream);
MI_API int32_t mi_kv_append_paged_f32_i8(const float *k_new, const float *v_new, int64_t row_stride,
                                         int8_t *kq_pool, float *ks_pool, int8_t *vq_pool, float *vs_pool,
                                         const int32_t *block_table, int64_t max_pages, int64_t page_size,
                                         const int32_t *pos, int64_t B, int64_t Hkv, int64_t D, void *stream);
/* a7 as the decode loop uses it: rotate (block 128 = D) and quantize the new token's key and value heads and
 * write codes and scale at token pos[b] of sequence b (int32 [B] in device memory; a sequence whose position is
 * outside [0, T_cap) is skipped).  Head h of sequence b is read at k_new + b*row_stride + h*D (floats), so
 * k_new/v_new may be slices of a fused QKV output (row_stride = its row length) or packed [B,Hkv,D]
 * (row_stride = Hkv*D).  Same arithmetic, bit for bit, as mi_fwht_quant_f32_i8 with K = block = 128. */
MI_API int32_t mi_kv_append_f32_i8(const float *k_new, const float *v_new, int64_t row_stride,
                                   int8_t *kq, float *ks, int8_t *vq, float *vs, const int32_t *pos,
                                   int64_t B, int64_t Hkv, int64_t D, int64_t T_cap, void *stream);
/* ---- the same attention over a cache stored in the two layouts the int8 matrix instruction loads straight from
 * memory (1 KB contiguous per wave instruction, nothing converted or transposed on the way):
 *   kt int8 [B, Hkv, T_cap/16, 8, 16, 16]  tile of 16 tokens: byte (c, t % 16, e) = code 16*c + e of token t
 *   vt int8 [B, Hkv, T_cap/64, 8, 4, 16, 16]  block of 64 tokens, transposed, in 16 x 16 pieces:
 *                                          byte (d / 16, (t % 64) / 16, d % 16, t % 16) = code d of token t
 * ks, vs fp32 [B, Hkv, T_cap] as above (16-byte aligned); T_cap % 64 == 0.  Both products of the attention run on
 * the int8 matrix pipe.  The softmax weights times the V scales enter the second one as 28-bit fixed-point numbers:
 * w_t = exp2(s_t - m) * vs_t is rounded to the nearest multiple of u = vmax * 2^-28, vmax the largest V scale among
 * the tokens of one split (at most 1024 of them), so a token whose V scale is vmax / r keeps 28 - log2(r) bits of
 * its weight.  Against the fp32 accumulation of the row-major kernel an output element therefore differs by at most
 * (tokens of the split) * 127 * u / 2 per split before the division by the softmax sum (which is >= 1), i.e. by
 * T * 127 * 2^-29 * vmax in all (a worst case with every rounding the same way): invisible while the V scales of a split lie within
 * two or three decades of each other (what a Hadamard-rotated cache holds), and a loss of precision that grows
 * with the spread beyond that.  This is the fast layout, and the one the decode-layer chain uses.  seq_len may be NULL (every sequence holds T_max tokens).  Workspace:
 * mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T_max) (one query serves both layouts).  Bytes that belong to tokens
 * at or past a sequence's length are never used (they may hold anything).  No upstream counterpart. */
MI_API int32_t mi_gqa_decode_attn_tiled(const float *q, const int8_t *kt, const float *ks,
                                        const int8_t *vt, const float *vs, float *o,
                                        int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T_cap,
                                        const int32_t *seq_len, int64_t T_max, int32_t out_rotated,
                                        void *workspace, int64_t workspace_bytes, void *stream);
/* ... with the merge fused with the output projection's row quantizer, as mi_gqa_decode_attn_cache_quant_i8. */
MI_API int32_t mi_gqa_decode_attn_tiled_quant_i8(const float *q, const int8_t *kt, const float *ks,
                                                 const int8_t *vt, const float *vs, float *o_rot,
                                                 int8_t *oq, float *oscale,
                                                 int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T_cap,
                                                 const int32_t *seq_len, int64_t T_max,
                                                 void *workspace, int64_t workspace_bytes, void *stream);
/* ... and with the output projection behind it, as one call: y fp32 [B, N] = the attention rows of a token (Hq*D
 * values in the rotated basis of V, quantized as one row) contracted with prepared projection weights qw int8
 * [N, Hq*D], sw fp32 [N] (rotated along K with block D), N % 16 == 0, Hq <= 64.  The values are those of
 * mi_gqa_decode_attn_tiled_quant_i8 followed by mi_w8a8_gemm_dequant_f32, bit for bit; what differs is the division
 * of the work for ONE token (B == 1, Hq*D in {2048, 4096}): the merge then runs over many workgroups and leaves the
 * fp32 row, and the projection's GEMV quantizes that row in its own prologue (three launches, none of which reads
 * every split's partials through one compute unit).  o_rot (optional, fp32 [B,Hq,D]) receives the merged row.
 * Workspace: mi_gqa_decode_attn_linear_workspace_bytes(B, Hq, Hkv, D, T_max).  It starts with the merged rows
 * (fp32, B*Hq*D*4 bytes), their codes (int8 [B, Hq*D]) and their scales (fp32 [B]), each area rounded up to 256
 * bytes - a caller may read them there after the call - and the attention's own workspace follows.  No upstream
 * counterpart. */
MI_API int64_t mi_gqa_decode_attn_linear_workspace_bytes(int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T);
MI_API int32_t mi_gqa_decode_attn_tiled_linear_f32(const float *q, const int8_t *kt, const float *ks,
                                                   const int8_t *vt, const float *vs, float *o_rot,
                                                   const int8_t *qw, const float *sw, float *y,
                                                   int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T_cap,
                                                   const int32_t *seq_len, int64_t T_max, int64_t N,
                                                   void *workspace, int64_t workspace_bytes, void *stream);
/* Row-major codes [rows, src_stride tokens, 128] (rows = B*Hkv) -> the tiled layouts, first T tokens of every row
 * (the rest of the last 64-token block touched is zero-filled); either pair (kq, kt) / (vq, vt) may be NULL.  For
 * caches that were quantized in one go (prefill) with mi_fwht_quant_f32_i8. */
MI_API int32_t mi_kv_tiled_from_rows_i8(const int8_t *kq, const int8_t *vq, int8_t *kt, int8_t *vt,
                                        int64_t rows, int64_t T, int64_t src_stride, int64_t T_cap, void *stream);
/* mi_kv_append_f32_i8 and mi_rope_kv_append_f32_i8 for these layouts (same arithmetic, same codes and scales, at
 * the tiled places of token pos[b]). */
MI_API int32_t mi_kv_append_tiled_f32_i8(const float *k_new, const float *v_new, int64_t row_stride,
                                         int8_t *kt, float *ks, int8_t *vt, float *vs, const int32_t *pos,
                                         int64_t B, int64_t Hkv, int64_t D, int64_t T_cap, void *stream);
MI_API int32_t mi_rope_kv_append_tiled_f32_i8(const float *qkv, int64_t row_stride, const float *rope_cos,
                                              const float *rope_sin, float *q_out, int8_t *kt, float *ks,
                                              int8_t *vt, float *vs, const int32_t *pos,
                                              int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T_cap,
                                              void *stream);
/* Paged form of the tiled cache: pools of 64-token pages.  A page holds, per kv head, one 8 KB key block (four
 * 16-token tiles in the layout above) and one 8 KB transposed value block, plus 64 key and 64 value scales:
 *   kt_pool, vt_pool int8 [pages, Hkv, 8192];  ks_pool, vs_pool fp32 [pages, Hkv, 64]
 * Tokens [64 i, 64 i + 64) of sequence b live in page block_table[b * max_pages + i] (int32 in device memory; every
 * entry that covers a token below seq_len[b], resp. the position being appended, must be a valid page of the pool:
 * the kernels cannot check it; entries behind a sequence's last block may hold anything).  The attention kernel's
 * loads stay 1 KB contiguous and a block costs it one scalar table look-up; arithmetic and results are those of the
 * dense tiled layout, bit for bit.  seq_len is required.  No upstream counterpart: the allocator idea of one slab
 * handing out fixed pieces (threading/numa_arena.mojo:40-55) applied to the cache. */
MI_API int32_t mi_gqa_decode_attn_tiled_paged(const float *q, const int8_t *kt_pool, const float *ks_pool,
                                              const int8_t *vt_pool, const float *vs_pool, float *o,
                                              const int32_t *block_table, int64_t max_pages,
                                              int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                                              const int32_t *seq_len, int64_t T_max, int32_t out_rotated,
                                              void *workspace, int64_t workspace_bytes, void *stream);
MI_API int32_t mi_gqa_decode_attn_tiled_paged_quant_i8(const float *q, const int8_t *kt_pool, const float *ks_pool,
                                                       const int8_t *vt_pool, const float *vs_pool, float *o_rot,
                                                       int8_t *oq, float *oscale,
                                                       const int32_t *block_table, int64_t max_pages,
                                                       int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                                                       const int32_t *seq_len, int64_t T_max,
                                                       void *workspace, int64_t workspace_bytes, void *stream);
MI_API int32_t mi_kv_append_tiled_paged_f32_i8(const float *k_new, const float *v_new, int64_t row_stride,
                                               int8_t *kt_pool, float *ks_pool, int8_t *vt_pool, float *vs_pool,
                                               const int32_t *block_table, int64_t max_pages, const int32_t *pos,
                                               int64_t B, int64_t Hkv, int64_t D, void *stream);
MI_API int32_t mi_rope_kv_append_tiled_paged_f32_i8(const float *qkv, int64_t row_stride, const float *rope_cos,
                                                    const float *rope_sin, float *q_out,
                                                    int8_t *kt_pool, float *ks_pool, int8_t *vt_pool, float *vs_pool,
                                                    const int32_t *block_table, int64_t max_pages, const int32_t *pos,
                                                    int64_t B, int64_t Hq, int64_t Hkv, int64_t D, void *stream);
/* Gate helper for the tiled layout: the split kernel of mi_gqa_decode_attn_tiled alone, which also writes out the
 * int8 query codes [B,Hq,D], their scales [B,Hq] and the raw int32 scores [B,Hq,T] it works from (no merge, no o;
 * every sequence holds T tokens). */
MI_API int32_t mi_gqa_decode_scores_tiled_i32(const float *q, const int8_t *kt, const float *ks,
                                              const int8_t *vt, const float *vs,
                                              int8_t *qq, float *sq, int32_t *dots,
                                              int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T_cap, int64_t T,
                                              void *workspace, int64_t workspace_bytes, void *stream);
/* Gate helper: runs the same split kernel and also writes out the int8 query
 * codes [B,Hq,D], their scales [B,Hq] and the raw int32 scores [B,Hq,T] it
 * works from (no merge, no o). */
MI_API int32_t mi_gqa_decode_scores_i32(const float *q, const int8_t *kq, const float *ks,
                                        const int8_t *vq, const float *vs,
                                        int8_t *qq, float *sq, int32_t *dots,
                                        int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t T,
                                        void *workspace, int64_t workspace_bytes, void *stream);

/* ---- a9: MoE router: logits = x . wr^T in a fixed fp32 order, top-k on the
 * logits (ties to the lower expert), weights = softmax over the k picks.
 * x fp32 [T,H], wr fp32 [E,H] -> idx int32 [T,topk], w fp32 [T,topk].
 * H % 256 == 0, E % 16 == 0, E <= 256, topk <= 8. */
MI_API int64_t mi_moe_route_workspace_bytes(int64_t T, int64_t E);   /* the fp32 logits [T,E] */
MI_API int32_t mi_moe_route(const float *x, const float *wr, int32_t *idx, float *w,
                            int64_t T, int64_t H, int64_t E, int32_t topk,
                            void *workspace, int64_t workspace_bytes, void *stream);
/* ---- a10: stable grouping of the T*topk (token,slot) pairs by expert.
 * idx int32 [T,topk] -> perm int32 [T*topk] (perm[pos] = pair = token*topk+slot),
 * seg_off int32 [E+1].  2 * E * ceil(T/32) + E + 1 <= 36864 (the bitmaps live in LDS). */
MI_API int32_t mi_moe_dispatch(const int32_t *idx, int32_t *perm, int32_t *seg_off,
                               int64_t T, int64_t E, int32_t topk, void *stream);
/* ---- a11: grouped expert SwiGLU FFN over expert-sorted segments.
 * x fp32 [T,H]; idx,w [T,topk]; wg,wu int8 [E,I,H] + sg,su fp32 [E,I];
 * wd int8 [E,H,I] + sd fp32 [E,H]; y fp32 [T,H].
 * H % 128 == 0 (input block 128), I % 256 == 0 (inner block 256).
 * idx as mi_moe_route writes it: a token lists an expert at most once (a repeated expert would be dispatched once:
 * the kernels cannot check it).  A slot whose index lies outside [0, E) is skipped: it contributes 0 to y. */
MI_API int64_t mi_moe_ffn_workspace_bytes(int64_t T, int64_t H, int64_t I, int64_t E, int32_t topk);
MI_API int32_t mi_moe_ffn(const float *x, const int32_t *idx, const float *w,
                          const int8_t *wg, const float *sg, const int8_t *wu, const float *su,
                          const int8_t *wd, const float *sd, float *y,
                          int64_t T, int64_t H, int64_t I, int64_t E, int32_t topk,
                          void *workspace, int64_t workspace_bytes, void *stream);
/* Byte offsets into the mi_moe_ffn workspace, for gates that inspect the
 * intermediates: which = 0 qx int8[T,H], 1 sx f32[T], 2 perm i32[T*topk],
 * 3 seg_off i32[E+1], 4 h f32[T*topk,I] (sorted order), 5 hq int8[T*topk,I],
 * 6 hs f32[T*topk], 7 out f32[T*topk,H] (pair order), 8 idx i32[T,topk],
 * 9 w f32[T,topk] and 10 router logits f32[T,E] (8-10 filled by mi_moe_layer only).  Negative on error. */
MI_API int64_t mi_moe_ffn_workspace_offset(int32_t which, int64_t T, int64_t H, int64_t I,
                                           int64_t E, int32_t topk);
/* Router + dispatch + FFN in one call (routing results land in the workspace). */
MI_API int32_t mi_moe_layer(const float *x, const float *wr,
                            const int8_t *wg, const float *sg, const int8_t *wu, const float *su,
                            const int8_t *wd, const float *sd, float *y,
                            int64_t T, int64_t H, int64_t I, int64_t E, int32_t topk,
                            void *workspace, int64_t workspace_bytes, void *stream);
MI_API int64_t mi_moe_layer_workspace_bytes(int64_t T, int64_t H, int64_t I, int64_t E, int32_t topk);

/* ---- the fp32 operators between the int8 kernels of one decoder layer (decode step).  No upstream
 * counterpart (upstream holds no model code); they chain the entry points above into
 * RMSNorm -> QKV -> rotary + cache append -> attention -> O -> RMSNorm -> gate|up -> SwiGLU -> down.
 * RMSNorm: h = x (+ residual, then also written to h_out); y = (h * r) * g, r = 1/sqrt(mean(h^2) + eps).
 * x, residual, h_out, y fp32 [M,H]; g fp32 [H]; H % 4 == 0, H <= 16384. */
MI_API int32_t mi_rmsnorm_f32(const float *x, const float *residual, const float *g, float eps,
                              float *h_out, float *y, int64_t M, int64_t H, void *stream);
/* One decode token per sequence.  qkv fp32: row b = [Hq query heads | Hkv key heads | Hkv value heads] x D, rows
 * row_stride floats apart (the output of a fused QKV projection).  Query and key heads get the rotary embedding
 * of position pos[b]: pairs (i, i + D/2), x'[i] = x[i]*cos - x[i+D/2]*sin, x'[i+D/2] = x[i+D/2]*cos + x[i]*sin
 * with cos/sin = rope_cos/rope_sin[pos[b]][i] (fp32 [T_cap, D/2] tables of the caller).  Queries leave packed
 * in q_out fp32 [B,Hq,D] (what the attention entry points take); keys (after the embedding) and values are
 * rotated (block D) and quantized exactly as mi_kv_append_f32_i8 does and stored at token pos[b] of the cache.
 * A sequence whose position is outside [0, T_cap) writes nothing (its q_out rows keep what they held).  D == 128. */
MI_API int32_t mi_rope_kv_append_f32_i8(const float *qkv, int64_t row_stride, const float *rope_cos,
                                        const float *rope_sin, float *q_out, int8_t *kq, float *ks, int8_t *vq,
                                        float *vs,
                                        const int32_t *pos, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                                        int64_t T_cap, void *stream);
/* h[m,n] = silu(gate_up[m,n]) * gate_up[m,I+n]; gate_up fp32 [M,2I] (one projection of N = 2I), h fp32 [M,I]. */
MI_API int32_t mi_swiglu_f32(const float *gate_up, float *h, int64_t M, int64_t I, void *stream);
/* The two row operators above fused with the rotate + quantize prologue (mi_fwht_quant_f32_i8) of the linear that
 * consumes them: codes int8 [M,H] (resp. [M,I]) and scales fp32 [M] go straight to mi_w8a8_gemm_dequant_f32.
 * The arithmetic per element is that of the separate calls in the same order, and the sum of squares is taken in
 * an order that depends on the row alone: one token gives the same codes whatever M it is batched in, here and in
 * mi_rmsnorm_linear_f32, and they are the codes mi_fwht_quant_f32_i8 gives on the row y_out receives.
 * (mi_rmsnorm_f32 sums the squares in another order: its row may differ from y_out in the last bit.)  y_out / h_out of the activated row are optional (NULL: the
 * fp32 row is never written); with a residual, h_out (the sum) is required as above.  H, I % block == 0. */
MI_API int32_t mi_rmsnorm_quant_f32_i8(const float *x, const float *residual, const float *g, float eps,
                                       float *h_out, float *y_out, int8_t *q, float *scale,
                                       int64_t M, int64_t H, int32_t block, void *stream);
MI_API int32_t mi_swiglu_quant_f32_i8(const float *gate_up, float *h_out, int8_t *q, float *scale,
                                      int64_t M, int64_t I, int32_t block, void *stream);
/* (residual +) RMSNorm + rotate + quantize + W8A8 contraction + dequant as one call: y = linear(rmsnorm(x (+ residual))).
 * For one token and K in {2048, 4096} (block 128) it is ONE kernel (the GEMV normalizes and quantizes the row
 * itself); any other shape runs mi_rmsnorm_quant_f32_i8 and the contraction.  workspace as for mi_w8a8_linear_f32
 * (it receives the codes and the scale); h_out (the residual sum, required with a residual) and xn_out (the
 * normalized row, optional) as in mi_rmsnorm_quant_f32_i8. */
MI_API int32_t mi_rmsnorm_linear_f32(const float *x, const float *residual, const float *g, float eps,
                                     float *h_out, float *xn_out, const int8_t *qw, const float *sw, float *y,
                                     int64_t M, int64_t N, int64_t K, int32_t block,
                                     void *workspace, int64_t workspace_bytes, void *stream);
/* out = a + b over n floats (n % 4 == 0): the residual add that closes the layer. */
MI_API int32_t mi_add_f32(const float *a, const float *b, float *out, int64_t n, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355_INT8_H */
