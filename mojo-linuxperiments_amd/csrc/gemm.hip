// C ABI of the W8A8 contraction: argument checks and the choice between the
// skinny weight-streaming kernel (M <= 64) and the LDS-tiled MFMA kernel.
#include <atomic>

#include "common.h"

namespace mi {
template <bool DEQ>
int32_t launch_skinny(const int8_t *, const float *, const int8_t *, const float *, int32_t *, float *, int64_t,
                      int64_t, int64_t, hipStream_t);
template <bool DEQ>
int32_t launch_tiled(const int8_t *, const float *, const int8_t *, const float *, int32_t *, float *, int64_t,
                     int64_t, int64_t, hipStream_t);

int32_t launch_linear_fused(const float *, const int8_t *, const float *, float *, int8_t *, float *, int64_t, int64_t,
                            int64_t, hipStream_t, bool);
int32_t launch_norm_linear_fused(const float *, const float *, const float *, float, float *, float *, const int8_t *,
                                 const float *, float *, int8_t *, float *, int64_t, int64_t, int64_t, hipStream_t);

__global__ void k_dequant(const int32_t *__restrict__ acc, const float *__restrict__ sx,
                          const float *__restrict__ sw, float *__restrict__ y, int64_t M, int64_t N)
{
    const int64_t total = M * N;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t m = i / N, n = i - m * N;
        y[i] = ((float)acc[i] * sx[m]) * sw[n];
    }
}

static int32_t check_gemm(const void *qx, const void *qw, const void *out, int64_t M, int64_t N, int64_t K)
{
    if (!qx || !qw || !out || M < 0 || N <= 0 || K <= 0) return MI_EINVAL;
    if (K % 128 || N % 16) return MI_EINVAL;
    if (M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL) return MI_ERANGE;
    if ((int64_t)127 * 127 * K > 0x7fffffffLL) return MI_ERANGE;  // int32 accumulator bound
    if (!aligned16(qx) || !aligned16(qw) || !aligned16(out)) return MI_EINVAL;
    return MI_OK;
}

int32_t gemm_dispatch(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw, int32_t *acc, float *y,
                      int64_t M, int64_t N, int64_t K, hipStream_t s)
{
    if (M == 0) return MI_OK;
    if (y) {
        return M <= 64 ? launch_skinny<true>(qx, sx, qw, sw, nullptr, y, M, N, K, s)
                       : launch_tiled<true>(qx, sx, qw, sw, nullptr, y, M, N, K, s);
    }
    return M <= 64 ? launch_skinny<false>(qx, nullptr, qw, nullptr, acc, nullptr, M, N, K, s)
                   : launch_tiled<false>(qx, nullptr, qw, nullptr, acc, nullptr, M, N, K, s);
}
}  // namespace mi

using namespace mi;

extern "C" int32_t mi_w8a8_gemm_i32(const int8_t *qx, const int8_t *qw, int32_t *acc, int64_t M, int64_t N,
                                    int64_t K, void *stream)
{
    int32_t rc = check_gemm(qx, qw, acc, M, N, K);
    if (rc) return rc;
    return gemm_dispatch(qx, nullptr, qw, nullptr, acc, nullptr, M, N, K, as_stream(stream));
}

extern "C" int32_t mi_w8a8_gemm_dequant_f32(const int8_t *qx, const float *sx, const int8_t *qw, const float *sw,
                                            float *y, int64_t M, int64_t N, int64_t K, void *stream)
{
    int32_t rc = check_gemm(qx, qw, y, M, N, K);
    if (rc) return rc;
    if (!sx || !sw || !aligned4(sx) || !aligned16(sw)) return MI_EINVAL;
    return gemm_dispatch(qx, sx, qw, sw, nullptr, y, M, N, K, as_stream(stream));
}

extern "C" int32_t mi_dequant_i32_f32(const int32_t *acc, const float *sx, const float *sw, float *y, int64_t M,
                                      int64_t N, void *stream)
{
    if (!acc || !sx || !sw || !y || M < 0 || N <= 0) return MI_EINVAL;
    if (M == 0) return MI_OK;
    int64_t blocks = (M * N + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(k_dequant, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), acc, sx, sw, y, M, N);
    return launch_status();
}

static int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// do the byte ranges [a, a + bytes) and [b, b + bytes) share a byte (null = no range)
static bool overlaps(const void *a, const void *b, int64_t bytes)
{
    if (!a || !b) return false;
    const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
    return pa < pb + (uintptr_t)bytes && pb < pa + (uintptr_t)bytes;
}

extern "C" int64_t mi_w8a8_linear_workspace_bytes(int64_t M, int64_t N, int64_t K)
{
    (void)N;
    if (M < 0 || K <= 0) return MI_EINVAL;
    return align_up(M * K, 256) + align_up(M * 4, 256);
}

extern "C" int32_t mi_rmsnorm_linear_f32(const float *x, const float *residual, const float *g, float eps,
                                         float *h_out, float *xn_out, const int8_t *qw, const float *sw, float *y,
                                         int64_t M, int64_t N, int64_t K, int32_t block, void *workspace,
                                         int64_t workspace_bytes, void *stream)
{
    if (!workspace || !aligned16(workspace)) return MI_EINVAL;
    if (workspace_bytes < mi_w8a8_linear_workspace_bytes(M, N, K)) return MI_ENOSPC;
    int8_t *qx = static_cast<int8_t *>(workspace);
    float *sx = reinterpret_cast<float *>(qx + align_up(M * K, 256));
    int32_t rc = check_gemm(qx, qw, y, M, N, K);
    if (rc) return rc;
    if (!x || !g || !sw || !aligned16(sw) || !aligned16(x) || !aligned16(g) || !(eps >= 0.0f)) return MI_EINVAL;
    if (residual && (!h_out || !aligned16(residual) || !aligned16(h_out))) return MI_EINVAL;
    if (xn_out && !aligned16(xn_out)) return MI_EINVAL;
    // The one-kernel form reads x and residual in every workgroup while one of them writes h_out / xn_out: a caller
    // that updates its residual stream in place (h_out or xn_out overlapping x or residual) takes the two-kernel
    // form, whose row operator reads each element before it writes it.
    const int64_t row_bytes = M * K * 4;
    const bool in_place = overlaps(h_out, x, row_bytes) || overlaps(h_out, residual, row_bytes) ||
                          overlaps(xn_out, x, row_bytes) || overlaps(xn_out, residual, row_bytes);
    if (M == 1 && block == 128 && !in_place) {
        rc = launch_norm_linear_fused(x, residual, g, eps, h_out, xn_out, qw, sw, y, qx, sx, M, N, K, as_stream(stream));
        if (rc != MI_EINVAL) return rc;
    }
    rc = mi_rmsnorm_quant_f32_i8(x, residual, g, eps, h_out, xn_out, qx, sx, M, K, block, stream);
    if (rc) return rc;
    return gemm_dispatch(qx, sx, qw, sw, nullptr, y, M, N, K, as_stream(stream));
}

// The linear once its activation codes (qx) and scales (sx) have a home: the caller's workspace or the static array.
static int32_t linear_with(const float *x, const int8_t *qw, const float *sw, float *y, int64_t M, int64_t N,
                           int64_t K, int32_t block, int8_t *qx, float *sx, void *stream)
{
    int32_t rc = check_gemm(qx, qw, y, M, N, K);
    if (rc) return rc;
    if (!x || !sw || !aligned16(sw)) return MI_EINVAL;
    if (M == 1 && block == 128 && aligned16(x)) {
        // decode: one kernel that quantizes its own activations (MI_EINVAL = shape not covered)
        rc = launch_linear_fused(x, qw, sw, y, qx, sx, M, N, K, as_stream(stream), true);
        if (rc != MI_EINVAL) return rc;
    }
    rc = mi_fwht_quant_f32_i8(x, qx, sx, M, K, block, stream);
    if (rc) return rc;
    return gemm_dispatch(qx, sx, qw, sw, nullptr, y, M, N, K, as_stream(stream));
}

extern "C" int32_t mi_w8a8_linear_f32(const float *x, const int8_t *qw, const float *sw, float *y, int64_t M,
                                      int64_t N, int64_t K, int32_t block, void *workspace,
                                      int64_t workspace_bytes, void *stream)
{
    if (!workspace || !aligned16(workspace)) return MI_EINVAL;
    if (workspace_bytes < mi_w8a8_linear_workspace_bytes(M, N, K)) return MI_ENOSPC;
    int8_t *qx = static_cast<int8_t *>(workspace);
    float *sx = reinterpret_cast<float *>(qx + align_up(M * K, 256));
    return linear_with(x, qw, sw, y, M, N, K, block, qx, sx, stream);
}

// ---- the same linear for callers that cannot allocate (code under graph capture, serving loops, harnesses that
// forbid hipMalloc): the activation codes and scales live in a static device array instead of a caller workspace.
// Every device the library runs on holds its own copy of the array, at its own address, until the process ends.
static constexpr int64_t NOALLOC_CODE_BYTES = 8ll << 20;   // M * K activation codes
static constexpr int64_t NOALLOC_MAX_ROWS = 8192;          // M scales
static constexpr int64_t NOALLOC_BYTES = NOALLOC_CODE_BYTES + NOALLOC_MAX_ROWS * 4;
static __device__ __align__(256) unsigned char scratch[NOALLOC_BYTES];

// In host code `scratch` is only a handle for the symbol: the array's device address is asked for once per device,
// with that device current, and every later use goes through the pointer kept here.
static constexpr int NOALLOC_MAX_DEVICES = 64;
static std::atomic<unsigned char *> g_scratch_ptr[NOALLOC_MAX_DEVICES];

namespace mi {
int32_t linear_scratch_bind(int device, unsigned char **out)   // `device` must be the current device
{
    if (device < 0 || device >= NOALLOC_MAX_DEVICES) return MI_ERANGE;
    unsigned char *p = g_scratch_ptr[device].load(std::memory_order_acquire);
    if (!p) {
        void *sym = nullptr;
        MI_HIP(hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)));
        if (!sym) return MI_EIO;
        p = static_cast<unsigned char *>(sym);
        g_scratch_ptr[device].store(p, std::memory_order_release);   // a race stores the same address twice
    }
    if (out) *out = p;
    return MI_OK;
}
}  // namespace mi

extern "C" int64_t mi_w8a8_linear_noalloc_max_codes(void) { return NOALLOC_CODE_BYTES; }
extern "C" int64_t mi_w8a8_linear_noalloc_max_rows(void) { return NOALLOC_MAX_ROWS; }

extern "C" int32_t mi_w8a8_linear_f32_noalloc(const float *x, const int8_t *qw, const float *sw, float *y, int64_t M,
                                              int64_t N, int64_t K, int32_t block, void *stream)
{
    if (M < 0 || K <= 0) return MI_EINVAL;
    if (M > NOALLOC_MAX_ROWS || K > NOALLOC_CODE_BYTES || M * K > NOALLOC_CODE_BYTES) return MI_ERANGE;
    int device = -1;
    MI_HIP(hipGetDevice(&device));
    unsigned char *base = nullptr;
    int32_t rc = linear_scratch_bind(device, &base);   // already bound when a context was created on this device
    if (rc) return rc;
    int8_t *qx = reinterpret_cast<int8_t *>(base);
    float *sx = reinterpret_cast<float *>(base + NOALLOC_CODE_BYTES);
    // nothing in the array has to start at zero: the quantizer writes every code and scale the contraction reads
    return linear_with(x, qw, sw, y, M, N, K, block, qx, sx, stream);
}
