// What a grid-wide wait costs on this machine, and what the runtime's cooperative launch costs around it.
// A kernel of one workgroup per compute unit: every workgroup adds one to a counter in device memory and waits
// (bounded by the 100 MHz real-time clock, ending in a normal exit with an error flag) until all have.  Timed with
// events as a cooperative launch and as a plain launch, with and without the wait, eagerly and as a graph replay.
// Prints one JSON line.  Measurement tool only (bench.py --grid-wait-probe): nothing in the library uses it.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CK(x)                                                                                             \
    do {                                                                                                  \
        hipError_t e_ = (x);                                                                              \
        if (e_ != hipSuccess) {                                                                           \
            fprintf(stderr, "hip error %d (%s) at line %d\n", (int)e_, hipGetErrorString(e_), __LINE__); \
            exit(1);                                                                                      \
        }                                                                                                 \
    } while (0)

__global__ __launch_bounds__(512) void k_wait(unsigned *flag, unsigned *err, unsigned long long *ticks, unsigned expect,
                                              int do_wait)
{
    const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
    if (do_wait) {
        if (threadIdx.x == 0) {
            __hip_atomic_fetch_add(flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            unsigned v;
            do {
                v = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (__builtin_amdgcn_s_memrealtime() - t0 > 100000ull) {   // 1 ms: give up, say so, leave normally
                    *err = 1;
                    break;
                }
            } while (v < expect);
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) ticks[blockIdx.x] = __builtin_amdgcn_s_memrealtime() - t0;
}
__global__ void k_zero(unsigned *flag) { *flag = 0; }

struct Run {
    float event_us;
    double in_kernel_us;
};

int main()
{
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    int coop = 0, occ = 0;
    CK(hipDeviceGetAttribute(&coop, hipDeviceAttributeCooperativeLaunch, 0));
    CK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, k_wait, 512, 0));
    unsigned *flag, *err;
    unsigned long long *ticks;
    CK(hipMalloc(&flag, 4));
    CK(hipMalloc(&err, 4));
    CK(hipMalloc(&ticks, 8 * 4096));
    CK(hipMemset(err, 0, 4));
    hipStream_t s;
    CK(hipStreamCreate(&s));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    unsigned expect = (unsigned)cus;   // one workgroup per compute unit: within the occupancy checked above
    int do_wait = 1;
    void *args[] = {&flag, &err, &ticks, &expect, &do_wait};
    auto timed = [&](bool cooperative, int wait) {
        do_wait = wait;
        Run best = {1e9f, 0};
        for (int rep = 0; rep < 30; ++rep) {
            hipLaunchKernelGGL(k_zero, dim3(1), dim3(1), 0, s, flag);
            CK(hipEventRecord(e0, s));
            if (cooperative) CK(hipLaunchCooperativeKernel((const void *)k_wait, dim3(cus), dim3(512), args, 0, s));
            else hipLaunchKernelGGL(k_wait, dim3(cus), dim3(512), 0, s, flag, err, ticks, expect, do_wait);
            CK(hipEventRecord(e1, s));
            CK(hipStreamSynchronize(s));
            float ms;
            CK(hipEventElapsedTime(&ms, e0, e1));
            if (ms * 1e3f < best.event_us) {
                unsigned long long h[4096], mx = 0;
                CK(hipMemcpy(h, ticks, 8 * (size_t)cus, hipMemcpyDeviceToHost));
                for (int i = 0; i < cus; ++i) mx = h[i] > mx ? h[i] : mx;
                best = {ms * 1e3f, mx / 100.0};
            }
        }
        return best;
    };
    auto replay = [&](bool cooperative) {   // graph of (clear + kernel with wait), microseconds per replay, or -1
        do_wait = 1;
        hipGraph_t g;
        hipGraphExec_t ge;
        CK(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
        hipLaunchKernelGGL(k_zero, dim3(1), dim3(1), 0, s, flag);
        hipError_t ce = hipSuccess;
        if (cooperative) ce = hipLaunchCooperativeKernel((const void *)k_wait, dim3(cus), dim3(512), args, 0, s);
        else hipLaunchKernelGGL(k_wait, dim3(cus), dim3(512), 0, s, flag, err, ticks, expect, do_wait);
        const hipError_t ee = hipStreamEndCapture(s, &g);
        if (ce != hipSuccess || ee != hipSuccess) return -1.0f;
        CK(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0));
        float best = 1e9f;
        for (int rep = 0; rep < 6; ++rep) {
            CK(hipEventRecord(e0, s));
            for (int i = 0; i < 20; ++i) CK(hipGraphLaunch(ge, s));
            CK(hipEventRecord(e1, s));
            CK(hipStreamSynchronize(s));
            float ms;
            CK(hipEventElapsedTime(&ms, e0, e1));
            best = ms * 1e3f / 20 < best ? ms * 1e3f / 20 : best;
        }
        CK(hipGraphExecDestroy(ge));
        CK(hipGraphDestroy(g));
        return best;
    };
    const Run c0 = timed(true, 0), c1 = timed(true, 1), p0 = timed(false, 0), p1 = timed(false, 1);
    const float gc = replay(true), gp = replay(false);
    unsigned herr = 0;
    CK(hipMemcpy(&herr, err, 4, hipMemcpyDeviceToHost));
    printf("{\"grid_wide_wait\": {\"compute_units\": %d, \"cooperative_launch_supported\": %d, "
           "\"workgroups_of_512_per_unit\": %d, \"workgroups\": %d, "
           "\"cooperative_launch_us\": {\"empty\": %.2f, \"with_wait\": %.2f, \"longest_workgroup_with_wait\": %.2f}, "
           "\"plain_launch_us\": {\"empty\": %.2f, \"with_wait\": %.2f, \"longest_workgroup_with_wait\": %.2f}, "
           "\"graph_replay_clear_plus_wait_kernel_us\": {\"cooperative\": %.2f, \"plain\": %.2f}, "
           "\"waits_that_timed_out\": %u}}\n",
           cus, coop, occ, cus, c0.event_us, c1.event_us, c1.in_kernel_us, p0.event_us, p1.event_us, p1.in_kernel_us, gc, gp,
           herr);
    return herr ? 1 : 0;
}
