// What the int8 matrix pipe of this machine sustains when nothing else limits it: a loop of
// v_mfma_i32_16x16x64_i8 alone, operands in registers, no memory traffic inside the loop, on every SIMD of the chip,
// for about 3 ms a run, twelve runs in a row of which the last counts.  The published peak (5.0 POP/s dense) is the
// instruction's rate at the top clock; under a sustained matrix load the clock is set by the power limit, and how
// far it falls depends on how many bits the operands toggle.  This probe measures that ceiling, which a GEMM's
// roofline fraction has to be read against:
//   - one and two waves per SIMD (one wave cannot issue the instruction back to back at the pipe's full rate);
//   - operands all zero, and int8 codes drawn like rotated, quantized activations (normal, sigma 30, clipped to 127);
//   - with and without the LDS fragment reads of the 8 x 6 wave tile (14 ds_read_b128 to 48 matrix instructions).
//   - "loop_variants": two waves per SIMD, activation-like codes, with what a GEMM's stage adds to the loop: more
//     fragment reads (20 and 28 to 48 matrix instructions), direct-to-LDS loads from a small cache-resident buffer
//     (7 and 14 KB per wave and 48 instructions), and a workgroup barrier every 48 instructions.
// Prints one JSON line.  Measurement tool only: nothing in the library uses it.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <utility>
#include <vector>

typedef int v4i __attribute__((ext_vector_type(4)));
#define CK(x)                                                                        \
    do {                                                                             \
        hipError_t e_ = (x);                                                         \
        if (e_ != hipSuccess) {                                                      \
            fprintf(stderr, "hip error %d (%s) at line %d\n", (int)e_, hipGetErrorString(e_), __LINE__); \
            exit(1);                                                                 \
        }                                                                            \
    } while (0)

template <int LO>
__device__ __forceinline__ void mfma_acc(const v4i &a, const v4i &b)
{
    asm volatile("v_mfma_i32_16x16x64_i8 a[%c2:%c3], %0, %1, a[%c2:%c3]" ::"v"(a), "v"(b), "n"(LO), "n"(LO + 3));
}
template <int OFF>
__device__ __forceinline__ void rd(v4i &dst, unsigned addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
// direct-to-LDS load of 16 bytes per lane: global address = sbase + voff + OFF, LDS address = ldsaddr + OFF + 16 * lane
template <int OFF>
__device__ __forceinline__ void dma16(const void *sbase, unsigned voff, unsigned ldsaddr)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3"
                 :
                 : "v"(voff), "s"(sbase), "s"(ldsaddr), "n"(OFF)
                 : "memory", "m0");
}
template <int N, class F>
__device__ __forceinline__ void sfor(F &&f)
{
    if constexpr (N > 0) {
        sfor<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// 48 accumulators of four registers (a0..a191), 8 + 6 operand fragments: the register picture of the GEMM's wave tile
template <bool READS>
__global__ __launch_bounds__(512) void k_mfma_loop(const unsigned *__restrict__ codes, long long *__restrict__ ticks,
                                                   int iters)
{
    extern __shared__ __attribute__((aligned(16))) char smem[];
    asm volatile("" ::: "a0", "a31", "a63", "a95", "a127", "a159", "a191");
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    unsigned *l32 = reinterpret_cast<unsigned *>(smem);
    for (int q = threadIdx.x; q < 16384; q += blockDim.x) l32[q] = codes[(blockIdx.x & 15) * 16384 + q];
    __syncthreads();
    const unsigned base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void *)smem;
    const unsigned addr = base + wave * 8192 + lane * 16;
    v4i xa[8], wb[6];
    sfor<8>([&](auto I) { rd<decltype(I)::value * 1024>(xa[decltype(I)::value], addr); });
    sfor<6>([&](auto I) { rd<decltype(I)::value * 1024 + 512>(wb[decltype(I)::value], addr); });
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __syncthreads();
    const long long t0 = __builtin_amdgcn_s_memtime();
    for (int it = 0; it < iters; ++it) {
        sfor<48>([&](auto I) {
            constexpr int i = decltype(I)::value;
            mfma_acc<4 * i>(wb[i / 8], xa[i % 8]);
            if constexpr (READS) {
                // the same fragments again: 14 reads to 48 matrix instructions, behind the last use of the register
                if constexpr (i >= 40) rd<(i - 40) * 1024>(xa[i - 40], addr);
                if constexpr (i % 8 == 7 && i < 40) rd<(i / 8) * 1024 + 512>(wb[i / 8], addr);
                if constexpr (i == 47) rd<5 * 1024 + 512>(wb[5], addr);
            }
        });
        if (READS) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    asm volatile("s_nop 15\ns_nop 15" ::: "memory");
    const long long t1 = __builtin_amdgcn_s_memtime();
    if (lane == 0) ticks[blockIdx.x * 8 + wave] = t1 - t0;
}

// The loop of k_mfma_loop<true> with EXTRA more fragment reads per 48 matrix instructions (into a register nobody
// uses), DMA direct-to-LDS loads of 1 KB per wave (four cache-resident lines of the code buffer, written behind
// the fragment area), and, BAR = 1, a workgroup barrier after every 48 instructions.
template <int EXTRA, int DMA, int BAR>
__global__ __launch_bounds__(512) void k_mfma_mix(const unsigned *__restrict__ codes, long long *__restrict__ ticks,
                                                  int iters)
{
    extern __shared__ __attribute__((aligned(16))) char smem[];
    asm volatile("" ::: "a0", "a31", "a63", "a95", "a127", "a159", "a191");
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    unsigned *l32 = reinterpret_cast<unsigned *>(smem);
    for (int q = threadIdx.x; q < 16384; q += blockDim.x) l32[q] = codes[(blockIdx.x & 15) * 16384 + q];
    __syncthreads();
    const unsigned base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void *)smem;
    const unsigned addr = base + wave * 8192 + lane * 16;
    const unsigned dbase = __builtin_amdgcn_readfirstlane(base + 65536 + wave * 8192);
    const unsigned voff0 = (unsigned)(lane * 16 + (blockIdx.x & 15) * 65536);
    v4i xa[8], wb[6], junk;
    sfor<8>([&](auto I) { rd<decltype(I)::value * 1024>(xa[decltype(I)::value], addr); });
    sfor<6>([&](auto I) { rd<decltype(I)::value * 1024 + 512>(wb[decltype(I)::value], addr); });
    rd<0>(junk, addr);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __syncthreads();
    const long long t0 = __builtin_amdgcn_s_memtime();
    for (int it = 0; it < iters; ++it) {
        sfor<48>([&](auto I) {
            constexpr int i = decltype(I)::value;
            mfma_acc<4 * i>(wb[i / 8], xa[i % 8]);
            if constexpr (i >= 40) rd<(i - 40) * 1024>(xa[i - 40], addr);
            if constexpr (i % 8 == 7 && i < 40) rd<(i / 8) * 1024 + 512>(wb[i / 8], addr);
            if constexpr (i == 47) rd<5 * 1024 + 512>(wb[5], addr);
            if constexpr (EXTRA > 0 && i < 40 && (i * EXTRA / 40) != ((i + 1) * EXTRA / 40)) rd<(i % 8) * 1024>(junk, addr);
            if constexpr (DMA > 0 && i < 40 && (i * DMA / 40) != ((i + 1) * DMA / 40))
                dma16<(i % 4) * 1024>(codes, voff0, dbase);
        });
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (DMA) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (BAR) __builtin_amdgcn_s_barrier();
        asm volatile("" ::"v"(junk));
    }
    asm volatile("s_nop 15\ns_nop 15" ::: "memory");
    const long long t1 = __builtin_amdgcn_s_memtime();
    if (lane == 0) ticks[blockIdx.x * 8 + wave] = t1 - t0;
}

struct Result {
    double ns_per_mfma, tops, tick_mhz, ticks_per_mfma;
};

template <bool READS>
static Result run(const unsigned *codes, long long *ticks, int waves_per_simd, int cus)
{
    const int threads = 256 * waves_per_simd, iters = 4000 / waves_per_simd * 2;
    CK(hipFuncSetAttribute((const void *)k_mfma_loop<READS>, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    float ms = 0;
    for (int rep = 0; rep < 12; ++rep) {   // the last repetition counts: 35 ms of the same load lie before it
        CK(hipEventRecord(e0, 0));
        hipLaunchKernelGGL(k_mfma_loop<READS>, dim3(cus), dim3(threads), 64 * 1024, 0, codes, ticks, iters);
        CK(hipEventRecord(e1, 0));
        CK(hipDeviceSynchronize());
        CK(hipEventElapsedTime(&ms, e0, e1));
    }
    std::vector<long long> h((size_t)cus * 8);
    CK(hipMemcpy(h.data(), ticks, h.size() * sizeof(long long), hipMemcpyDeviceToHost));
    double mean = 0;
    for (int b = 0; b < cus; ++b)
        for (int w = 0; w < 4 * waves_per_simd; ++w) mean += (double)h[(size_t)b * 8 + w];
    mean /= (double)cus * 4 * waves_per_simd;
    const double per_simd = 48.0 * iters * waves_per_simd;
    Result r;
    r.ns_per_mfma = ms * 1e6 / per_simd;
    r.tops = 2.0 * 16 * 16 * 64 * per_simd * 4 * cus / (ms * 1e-3) / 1e12;
    r.tick_mhz = mean / (ms * 1e3);
    r.ticks_per_mfma = mean / per_simd;
    CK(hipEventDestroy(e0));
    CK(hipEventDestroy(e1));
    return r;
}

template <int EXTRA, int DMA, int BAR>
static void run_mix(const unsigned *codes, long long *ticks, int cus, bool first)
{
    const int iters = 4000;
    CK(hipFuncSetAttribute((const void *)k_mfma_mix<EXTRA, DMA, BAR>, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    float ms = 0;
    for (int rep = 0; rep < 8; ++rep) {
        CK(hipEventRecord(e0, 0));
        hipLaunchKernelGGL((k_mfma_mix<EXTRA, DMA, BAR>), dim3(cus), dim3(512), 128 * 1024, 0, codes, ticks, iters);
        CK(hipEventRecord(e1, 0));
        CK(hipDeviceSynchronize());
        CK(hipEventElapsedTime(&ms, e0, e1));
    }
    std::vector<long long> h((size_t)cus * 8);
    CK(hipMemcpy(h.data(), ticks, h.size() * sizeof(long long), hipMemcpyDeviceToHost));
    double mean = 0;
    for (auto v : h) mean += (double)v;
    mean /= (double)h.size();
    const double per_simd = 48.0 * iters * 2;
    printf("%s{\"fragment_reads_per_48\": %d, \"direct_to_lds_kb_per_48\": %d, \"barrier_per_48\": %s, \"tops\": %.0f, "
           "\"ns_per_mfma\": %.2f, \"clock_ticks_per_mfma\": %.2f, \"clock_mhz\": %.0f}",
           first ? "" : ", ", 14 + EXTRA, DMA, BAR ? "true" : "false",
           2.0 * 16 * 16 * 64 * per_simd * 4 * cus / (ms * 1e-3) / 1e12, ms * 1e6 / per_simd, mean / per_simd, mean / (ms * 1e3));
    CK(hipEventDestroy(e0));
    CK(hipEventDestroy(e1));
}

int main()
{
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    // int8 codes like rotated, quantized activations: normal, sigma 30, clipped to +-127 (a fixed LCG + Box-Muller)
    std::vector<unsigned> gauss(17 * 16384), zeros(17 * 16384, 0u);   // (one more block: the mix loop's loads run past the 16th)
    unsigned long long st = 88172645463325252ull;
    auto uni = [&]() {
        st = st * 6364136223846793005ull + 1442695040888963407ull;
        return ((st >> 11) + 1) * (1.0 / 9007199254740994.0);
    };
    for (auto &w : gauss) {
        unsigned v = 0;
        for (int by = 0; by < 4; ++by) {
            const double g = std::sqrt(-2.0 * std::log(uni())) * std::cos(6.283185307179586 * uni());
            int c = (int)std::lrint(30.0 * g);
            c = c > 127 ? 127 : (c < -127 ? -127 : c);
            v |= ((unsigned)c & 255u) << (8 * by);
        }
        w = v;
    }
    unsigned *dcodes;
    long long *ticks;
    CK(hipMalloc(&dcodes, gauss.size() * 4));
    CK(hipMalloc(&ticks, (size_t)cus * 8 * sizeof(long long)));
    printf("{\"mfma_power_limited_peak\": {\"instruction\": \"v_mfma_i32_16x16x64_i8\", \"compute_units\": %d, "
           "\"published_peak_tops\": 5000, \"runs\": [",
           cus);
    bool first = true;
    for (int data = 0; data < 2; ++data) {
        CK(hipMemcpy(dcodes, data ? gauss.data() : zeros.data(), gauss.size() * 4, hipMemcpyHostToDevice));
        for (int reads = 0; reads < 2; ++reads)
            for (int wps = 1; wps <= 2; ++wps) {
                const Result r = reads ? run<true>(dcodes, ticks, wps, cus) : run<false>(dcodes, ticks, wps, cus);
                printf("%s{\"operands\": \"%s\", \"lds_fragment_reads\": %s, \"waves_per_simd\": %d, \"tops\": %.0f, "
                       "\"ns_per_mfma\": %.2f, \"clock_ticks_per_mfma\": %.2f, \"clock_mhz\": %.0f}",
                       first ? "" : ", ", data ? "normal codes, sigma 30" : "zeros", reads ? "true" : "false", wps, r.tops,
                       r.ns_per_mfma, r.ticks_per_mfma, r.tick_mhz);
                first = false;
            }
    }
    printf("], \"loop_variants\": [");
    run_mix<0, 0, 0>(dcodes, ticks, cus, true);
    run_mix<6, 0, 0>(dcodes, ticks, cus, false);
    run_mix<14, 0, 0>(dcodes, ticks, cus, false);
    run_mix<0, 7, 0>(dcodes, ticks, cus, false);
    run_mix<6, 7, 0>(dcodes, ticks, cus, false);
    run_mix<6, 14, 0>(dcodes, ticks, cus, false);
    run_mix<0, 0, 1>(dcodes, ticks, cus, false);
    run_mix<6, 7, 1>(dcodes, ticks, cus, false);
    printf("]}}\n");
    CK(hipFree(dcodes));
    CK(hipFree(ticks));
    return 0;
}
