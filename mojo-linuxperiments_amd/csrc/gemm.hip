// C ABI of the W8A8 contraction: argument checks and the choice between the
// skinny weight-streaming kernel (M <= 64) and the LDS-tiled MFMA kernel.
#include "common.h"

namespace mi {
template <bool DEQ>
int32_t launch_skinny(const int8_t *, const float *, const int8_t *, const float *, int32_t *, float *, int64_t,
                      int64_t, int64_t, hipStream_t);
template <bool DEQ>
int32_t launch_tiled(const int8_t *, const float *, const int8_t *, const float *, int32_t *, float *, int64_t,
                     int64_t, int64_t, hipStream_t);

int32_t launch_linear_fused(const float *, const int8_t *, const float *, float *, int8_t *, float *, int64_t, int64_t,
                            int64_t, hipStream_t);
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
    if (M == 1 && block == 128) {
        rc = launch_norm_linear_fused(x, residual, g, eps, h_out, xn_out, qw, sw, y, qx, sx, M, N, K, as_stream(stream));
        if (rc != MI_EINVAL) return rc;
    }
    rc = mi_rmsnorm_quant_f32_i8(x, residual, g, eps, h_out, xn_out, qx, sx, M, K, block, stream);
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
    int32_t rc = check_gemm(qx, qw, y, M, N, K);
    if (rc) return rc;
    if (!x || !sw || !aligned16(sw)) return MI_EINVAL;
    if (M == 1 && block == 128 && aligned16(x)) {
        // decode: one kernel that quantizes its own activations (MI_EINVAL = shape not covered)
        rc = launch_linear_fused(x, qw, sw, y, qx, sx, M, N, K, as_stream(stream));
        if (rc != MI_EINVAL) return rc;
    }
    rc = mi_fwht_quant_f32_i8(x, qx, sx, M, K, block, stream);
    if (rc) return rc;
    return gemm_dispatch(qx, sx, qw, sw, nullptr, y, M, N, K, as_stream(stream));
}
