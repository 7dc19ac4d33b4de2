// Runtime half of libmi355_int8.so: context, device arena, stream pool, gate,
// copies and events.  The arena follows NumaArena (threading/numa_arena.mojo:5-87)
// and the pool follows ThreadPool / MutexGate
// (threading/linux_threading.mojo:43-158, :174-198) in behaviour, with device
// memory, hipStreams and hipEvents in place of mmap/mbind, clone3 and futexes.
#include <sched.h>
#include <string.h>
#include <sys/syscall.h>
#include <unistd.h>

#include <new>

#include "common.h"

namespace mi {
thread_local int32_t g_last_hip_error = 0;

int32_t compute_units()
{
    static int32_t cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
        cached[dev] = v;
    }
    return cached[dev];
}

int32_t lds_limit()
{
    static int32_t cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 64 * 1024;
    if (cached[dev] == 0) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess || v <= 0) v = 64 * 1024;
        cached[dev] = v;
    }
    return cached[dev];
}

int32_t linear_scratch_bind(int device, unsigned char **out);   // gemm.hip: address of the static scratch array

__global__ void k_fill_u32(uint32_t *dst, uint32_t value, int64_t count)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) dst[i] = value;
}
}  // namespace mi

using namespace mi;

struct mi_ctx {
    int32_t device;
    int32_t cus;
    int64_t mem_bytes;
    char arch[64];
};

struct mi_arena {
    mi_ctx *ctx;
    uint8_t *base;
    int64_t size;
    int64_t offset;
    int64_t alignment;
    bool host;      // pinned host slab (staging) instead of device memory
    int32_t node;   // NUMA node a host slab is bound to, or -1
};

struct mi_slot {
    hipStream_t stream;
    hipEvent_t done;
    bool in_use;
};

struct mi_stream_pool {
    mi_ctx *ctx;
    int32_t capacity;
    mi_slot *slots;
};

struct mi_gate {
    hipEvent_t ev;
    bool released;
};

struct mi_event {
    hipEvent_t ev;
};

struct mi_graph {
    hipGraph_t graph;
    hipGraphExec_t exec;
};

extern "C" {

const char *mi_status_string(int32_t s)
{
    switch (s) {
    case MI_OK: return "ok";
    case MI_EIO: return "HIP runtime error";
    case MI_ENOMEM: return "out of memory";
    case MI_EBUSY: return "busy";
    case MI_ENODEV: return "no such gfx950 device";
    case MI_EINVAL: return "invalid argument";
    case MI_ENOSPC: return "workspace too small";
    case MI_ERANGE: return "size out of supported range";
    default: return "unknown status";
    }
}

int32_t mi_last_hip_error(void) { return g_last_hip_error; }
int32_t mi_abi_version(void) { return 1; }

int32_t mi_ctx_create(int32_t device, mi_ctx **out)
{
    if (!out) return MI_EINVAL;
    *out = nullptr;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || device < 0 || device >= n) return MI_ENODEV;
    MI_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    MI_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return MI_ENODEV;
    // the library's set-up call: look up this device's copy of the static scratch array now, so that
    // mi_w8a8_linear_f32_noalloc never has to on a caller's critical path
    int32_t rc = linear_scratch_bind(device, nullptr);
    if (rc) return rc;
    mi_ctx *c = new (std::nothrow) mi_ctx;
    if (!c) return MI_ENOMEM;
    c->device = device;
    c->cus = prop.multiProcessorCount;
    c->mem_bytes = (int64_t)prop.totalGlobalMem;
    strncpy(c->arch, prop.gcnArchName, sizeof(c->arch) - 1);
    c->arch[sizeof(c->arch) - 1] = 0;
    *out = c;
    return MI_OK;
}

int32_t mi_ctx_destroy(mi_ctx *ctx)
{
    if (!ctx) return MI_EINVAL;
    delete ctx;
    return MI_OK;
}

int32_t mi_ctx_device(const mi_ctx *ctx) { return ctx ? ctx->device : MI_EINVAL; }
int32_t mi_ctx_compute_units(const mi_ctx *ctx) { return ctx ? ctx->cus : MI_EINVAL; }
int64_t mi_ctx_memory_bytes(const mi_ctx *ctx) { return ctx ? ctx->mem_bytes : MI_EINVAL; }

int32_t mi_ctx_arch_name(const mi_ctx *ctx, char *buf, int64_t buf_len)
{
    if (!ctx || !buf || buf_len <= 0) return MI_EINVAL;
    strncpy(buf, ctx->arch, (size_t)buf_len - 1);
    buf[buf_len - 1] = 0;
    return MI_OK;
}

/* ---- arena ---------------------------------------------------------------- */

int32_t mi_arena_create(mi_ctx *ctx, int64_t size_bytes, int64_t alignment, mi_arena **out)
{
    if (!out) return MI_EINVAL;
    *out = nullptr;
    if (!ctx || size_bytes <= 0 || alignment <= 0 || (alignment & (alignment - 1))) return MI_EINVAL;
    MI_HIP(hipSetDevice(ctx->device));
    mi_arena *a = new (std::nothrow) mi_arena;
    if (!a) return MI_ENOMEM;
    void *p = nullptr;
    if (hipMalloc(&p, (size_t)size_bytes) != hipSuccess || !p) {
        (void)hipGetLastError();
        delete a;
        return MI_ENOMEM;
    }
    // fresh mmap pages read as zero; give device memory the same property
    const int64_t words = size_bytes / 4;
    if (words > 0) {
        hipLaunchKernelGGL(k_fill_u32, dim3(2048), dim3(256), 0, 0, (uint32_t *)p, 0u, words);
    }
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        (void)hipFree(p);
        delete a;
        return hip_fail(e);
    }
    a->ctx = ctx;
    a->base = (uint8_t *)p;
    a->size = size_bytes;
    a->offset = 0;
    a->alignment = alignment;
    a->host = false;
    a->node = -1;
    *out = a;
    return MI_OK;
}

// Pinned host slab for staging, bound to one NUMA node the way mmap_numa binds its mapping
// (threading/numa_arena.mojo:93-107): the calling thread's memory policy is MPOL_BIND to `numa_node` while the
// runtime allocates and the pages are touched, and is put back afterwards.  The runtime pins the pages itself
// (pinning memory that already exists is not available on every host, allocating pinned memory is).
int32_t mi_host_arena_create(mi_ctx *ctx, int64_t size_bytes, int64_t alignment, int32_t numa_node, mi_arena **out)
{
    if (!out) return MI_EINVAL;
    *out = nullptr;
    if (!ctx || size_bytes <= 0 || alignment <= 0 || (alignment & (alignment - 1))) return MI_EINVAL;
    if (numa_node < -1 || numa_node >= 64) return MI_EINVAL;
    MI_HIP(hipSetDevice(ctx->device));
    mi_arena *a = new (std::nothrow) mi_arena;
    if (!a) return MI_ENOMEM;
    constexpr int MPOL_DEFAULT_ = 0, MPOL_BIND_ = 2;
    bool bound = false;
    if (numa_node >= 0) {
        unsigned long mask = 1UL << numa_node;
        if (syscall(SYS_set_mempolicy, MPOL_BIND_, &mask, 65UL) != 0) { delete a; return MI_EINVAL; }
        bound = true;
    }
    void *p = nullptr;
    hipError_t e = hipHostMalloc(&p, (size_t)size_bytes, bound ? hipHostMallocNumaUser : hipHostMallocDefault);
    if (e == hipSuccess && p) memset(p, 0, (size_t)size_bytes);   // first touch under the policy; fresh pages read as zero
    if (bound) (void)syscall(SYS_set_mempolicy, MPOL_DEFAULT_, nullptr, 0UL);
    if (e != hipSuccess || !p) {
        (void)hipGetLastError();
        delete a;
        return MI_ENOMEM;
    }
    a->ctx = ctx;
    a->base = (uint8_t *)p;
    a->size = size_bytes;
    a->offset = 0;
    a->alignment = alignment;
    a->host = true;
    a->node = numa_node;
    *out = a;
    return MI_OK;
}

int32_t mi_arena_destroy(mi_arena *a)
{
    if (!a) return MI_EINVAL;
    hipError_t e = a->host ? hipHostFree(a->base) : hipFree(a->base);
    delete a;
    return e == hipSuccess ? MI_OK : hip_fail(e);
}

void *mi_arena_alloc(mi_arena *a, int64_t bytes)
{
    if (!a || bytes < 0) return nullptr;
    const int64_t aligned = (a->offset + a->alignment - 1) & ~(a->alignment - 1);
    if (aligned + bytes > a->size) return nullptr;
    a->offset = aligned + bytes;
    return a->base + aligned;
}

int64_t mi_arena_mark(const mi_arena *a) { return a ? a->offset : MI_EINVAL; }

int32_t mi_arena_reset_to(mi_arena *a, int64_t mark)
{
    if (!a) return MI_EINVAL;
    if (mark < 0 || mark > a->offset) return MI_EINVAL;
    a->offset = mark;
    return MI_OK;
}

int32_t mi_arena_reset(mi_arena *a)
{
    if (!a) return MI_EINVAL;
    a->offset = 0;
    return MI_OK;
}

int64_t mi_arena_remaining(const mi_arena *a) { return a ? a->size - a->offset : MI_EINVAL; }
int64_t mi_arena_used(const mi_arena *a) { return a ? a->offset : MI_EINVAL; }

int32_t mi_arena_verify_placement(const mi_arena *a)
{
    if (!a) return MI_EINVAL;
    if (a->offset == 0) return 1;
    if (a->host) {
        // numa_arena.mojo:80-87: ask the kernel which node holds the first page (move_pages with no target nodes).
        // Pinned pages are mapped by the GPU driver and the kernel's page query may not see them (status
        // -ENOENT): then what can be verified is that the slab is pinned host memory; its node is the policy
        // that was in force while it was allocated.
        void *page = a->base;
        int status = -1;
        if (syscall(SYS_move_pages, 0, 1UL, &page, nullptr, &status, 0) == 0 && status >= 0)
            return (a->node < 0 || status == a->node) ? 1 : 0;
        hipPointerAttribute_t hattr;
        MI_HIP(hipPointerGetAttributes(&hattr, a->base));
        return hattr.type == hipMemoryTypeHost ? 1 : 0;
    }
    hipPointerAttribute_t attr;
    MI_HIP(hipPointerGetAttributes(&attr, a->base));
    return (attr.type == hipMemoryTypeDevice && attr.device == a->ctx->device) ? 1 : 0;
}

/* ---- stream pool ------------------------------------------------------------ */

int32_t mi_stream_pool_create(mi_ctx *ctx, int32_t capacity, mi_stream_pool **out)
{
    if (!out) return MI_EINVAL;
    *out = nullptr;
    if (!ctx || capacity <= 0 || capacity > 1024) return MI_EINVAL;
    MI_HIP(hipSetDevice(ctx->device));
    mi_stream_pool *p = new (std::nothrow) mi_stream_pool;
    if (!p) return MI_ENOMEM;
    p->slots = new (std::nothrow) mi_slot[capacity];
    if (!p->slots) { delete p; return MI_ENOMEM; }
    p->ctx = ctx;
    p->capacity = capacity;
    for (int32_t i = 0; i < capacity; ++i) {
        p->slots[i].stream = nullptr;
        p->slots[i].done = nullptr;
        p->slots[i].in_use = false;
    }
    for (int32_t i = 0; i < capacity; ++i) {
        // default priority on purpose: every stream of the pool is equal
        hipError_t e = hipStreamCreateWithFlags(&p->slots[i].stream, hipStreamNonBlocking);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&p->slots[i].done, hipEventDisableTiming);
        if (e != hipSuccess) {
            for (int32_t j = 0; j <= i; ++j) {
                if (p->slots[j].done) (void)hipEventDestroy(p->slots[j].done);
                if (p->slots[j].stream) (void)hipStreamDestroy(p->slots[j].stream);
            }
            delete[] p->slots;
            delete p;
            return hip_fail(e);
        }
    }
    *out = p;
    return MI_OK;
}

static int32_t slot_poll(mi_slot &s)
{
    if (!s.in_use) return 0;
    hipError_t e = hipEventQuery(s.done);
    if (e == hipSuccess) { s.in_use = false; return 0; }
    if (e == hipErrorNotReady) { (void)hipGetLastError(); return 1; }
    return hip_fail(e);
}

int32_t mi_stream_pool_capacity(const mi_stream_pool *p) { return p ? p->capacity : MI_EINVAL; }

int32_t mi_stream_pool_begin(mi_stream_pool *p)
{
    if (!p) return MI_EINVAL;
    for (int32_t i = 0; i < p->capacity; ++i) {
        int32_t st = slot_poll(p->slots[i]);
        if (st < 0) return st;
        if (st == 0) return i;
    }
    return MI_EBUSY;
}

void *mi_stream_pool_stream(mi_stream_pool *p, int32_t slot)
{
    if (!p || slot < 0 || slot >= p->capacity) return nullptr;
    return (void *)p->slots[slot].stream;
}

int32_t mi_stream_pool_end(mi_stream_pool *p, int32_t slot)
{
    if (!p || slot < 0 || slot >= p->capacity) return MI_EINVAL;
    if (p->slots[slot].in_use) return MI_EBUSY;
    MI_HIP(hipEventRecord(p->slots[slot].done, p->slots[slot].stream));
    p->slots[slot].in_use = true;
    return MI_OK;
}

int32_t mi_stream_pool_in_use(mi_stream_pool *p, int32_t slot)
{
    if (!p || slot < 0 || slot >= p->capacity) return MI_EINVAL;
    return slot_poll(p->slots[slot]);
}

int32_t mi_stream_pool_wait_all(mi_stream_pool *p)
{
    if (!p) return MI_EINVAL;
    for (int32_t i = 0; i < p->capacity; ++i) {
        if (!p->slots[i].in_use) continue;
        MI_HIP(hipEventSynchronize(p->slots[i].done));
        p->slots[i].in_use = false;
    }
    return MI_OK;
}

int32_t mi_stream_pool_wait_any(mi_stream_pool *p)
{
    if (!p) return MI_EINVAL;
    for (;;) {
        bool any = false;
        for (int32_t i = 0; i < p->capacity; ++i) {
            if (!p->slots[i].in_use) continue;
            any = true;
            int32_t st = slot_poll(p->slots[i]);
            if (st < 0) return st;
            if (st == 0) return i;
        }
        if (!any) return -1;
        sched_yield();
    }
}

int32_t mi_stream_pool_destroy(mi_stream_pool *p)
{
    if (!p) return MI_EINVAL;
    for (int32_t i = 0; i < p->capacity; ++i) {
        int32_t st = slot_poll(p->slots[i]);
        if (st < 0) return st;
        if (st == 1) return MI_EBUSY;
    }
    for (int32_t i = 0; i < p->capacity; ++i) {
        (void)hipEventDestroy(p->slots[i].done);
        (void)hipStreamDestroy(p->slots[i].stream);
    }
    delete[] p->slots;
    delete p;
    return MI_OK;
}

/* ---- gate ---------------------------------------------------------------------- */

int32_t mi_gate_create(mi_ctx *ctx, mi_gate **out)
{
    if (!out) return MI_EINVAL;
    *out = nullptr;
    if (!ctx) return MI_EINVAL;
    MI_HIP(hipSetDevice(ctx->device));
    mi_gate *g = new (std::nothrow) mi_gate;
    if (!g) return MI_ENOMEM;
    hipError_t e = hipEventCreateWithFlags(&g->ev, hipEventDisableTiming);
    if (e != hipSuccess) { delete g; return hip_fail(e); }
    g->released = false;
    *out = g;
    return MI_OK;
}

int32_t mi_gate_destroy(mi_gate *g)
{
    if (!g) return MI_EINVAL;
    (void)hipEventDestroy(g->ev);
    delete g;
    return MI_OK;
}

int32_t mi_gate_release(mi_gate *g, void *stream)
{
    if (!g) return MI_EINVAL;
    MI_HIP(hipEventRecord(g->ev, as_stream(stream)));
    g->released = true;
    return MI_OK;
}

int32_t mi_gate_wait(mi_gate *g, void *stream)
{
    if (!g || !g->released) return MI_EINVAL;
    MI_HIP(hipStreamWaitEvent(as_stream(stream), g->ev, 0));
    return MI_OK;
}

int32_t mi_gate_wait_host(mi_gate *g)
{
    if (!g || !g->released) return MI_EINVAL;
    MI_HIP(hipEventSynchronize(g->ev));
    return MI_OK;
}

int32_t mi_gate_reset(mi_gate *g)
{
    if (!g) return MI_EINVAL;
    g->released = false;
    return MI_OK;
}

/* ---- graphs -------------------------------------------------------------------- */

int32_t mi_graph_capture_begin(void *stream)
{
    if (!stream) return MI_EINVAL;
    MI_HIP(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
    return MI_OK;
}

int32_t mi_graph_capture_end(void *stream, mi_graph **out)
{
    if (!out) return MI_EINVAL;
    *out = nullptr;
    if (!stream) return MI_EINVAL;
    hipGraph_t graph = nullptr;
    MI_HIP(hipStreamEndCapture(as_stream(stream), &graph));
    if (!graph) return MI_EINVAL;
    mi_graph *g = new (std::nothrow) mi_graph;
    if (!g) { (void)hipGraphDestroy(graph); return MI_ENOMEM; }
    g->graph = graph;
    hipError_t e = hipGraphInstantiate(&g->exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) { (void)hipGraphDestroy(graph); delete g; return hip_fail(e); }
    *out = g;
    return MI_OK;
}

int32_t mi_graph_launch(mi_graph *g, void *stream)
{
    if (!g) return MI_EINVAL;
    MI_HIP(hipGraphLaunch(g->exec, as_stream(stream)));
    return MI_OK;
}

int32_t mi_graph_destroy(mi_graph *g)
{
    if (!g) return MI_EINVAL;
    (void)hipGraphExecDestroy(g->exec);
    (void)hipGraphDestroy(g->graph);
    delete g;
    return MI_OK;
}

/* ---- copies, host staging, events ---------------------------------------------- */

int32_t mi_memcpy_h2d(void *dst, const void *src, int64_t bytes, void *stream)
{
    if (bytes < 0 || (bytes && (!dst || !src))) return MI_EINVAL;
    if (bytes == 0) return MI_OK;
    MI_HIP(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyHostToDevice, as_stream(stream)));
    return MI_OK;
}

int32_t mi_memcpy_d2h(void *dst, const void *src, int64_t bytes, void *stream)
{
    if (bytes < 0 || (bytes && (!dst || !src))) return MI_EINVAL;
    if (bytes == 0) return MI_OK;
    MI_HIP(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    return MI_OK;
}

int32_t mi_memcpy_d2d(void *dst, const void *src, int64_t bytes, void *stream)
{
    if (bytes < 0 || (bytes && (!dst || !src))) return MI_EINVAL;
    if (bytes == 0) return MI_OK;
    MI_HIP(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return MI_OK;
}

int32_t mi_fill_u32(void *dst, uint32_t value, int64_t count, void *stream)
{
    if (count < 0 || (count && !dst) || !aligned4(dst)) return MI_EINVAL;
    if (count == 0) return MI_OK;
    int64_t blocks = (count + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(k_fill_u32, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                       (uint32_t *)dst, value, count);
    return launch_status();
}

int32_t mi_stream_synchronize(void *stream)
{
    MI_HIP(hipStreamSynchronize(as_stream(stream)));
    return MI_OK;
}

void *mi_host_alloc(int64_t bytes)
{
    if (bytes <= 0) return nullptr;
    void *p = nullptr;
    if (hipHostMalloc(&p, (size_t)bytes, hipHostMallocDefault) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return p;
}

int32_t mi_host_free(void *p)
{
    if (!p) return MI_EINVAL;
    MI_HIP(hipHostFree(p));
    return MI_OK;
}

int32_t mi_event_create(mi_event **out)
{
    if (!out) return MI_EINVAL;
    *out = nullptr;
    mi_event *e = new (std::nothrow) mi_event;
    if (!e) return MI_ENOMEM;
    hipError_t r = hipEventCreate(&e->ev);
    if (r != hipSuccess) { delete e; return hip_fail(r); }
    *out = e;
    return MI_OK;
}

int32_t mi_event_destroy(mi_event *e)
{
    if (!e) return MI_EINVAL;
    (void)hipEventDestroy(e->ev);
    delete e;
    return MI_OK;
}

int32_t mi_event_record(mi_event *e, void *stream)
{
    if (!e) return MI_EINVAL;
    MI_HIP(hipEventRecord(e->ev, as_stream(stream)));
    return MI_OK;
}

int32_t mi_event_synchronize(mi_event *e)
{
    if (!e) return MI_EINVAL;
    MI_HIP(hipEventSynchronize(e->ev));
    return MI_OK;
}

int32_t mi_event_elapsed_ms(mi_event *start, mi_event *stop, float *ms)
{
    if (!start || !stop || !ms) return MI_EINVAL;
    MI_HIP(hipEventElapsedTime(ms, start->ev, stop->ev));
    return MI_OK;
}

}  // extern "C"
