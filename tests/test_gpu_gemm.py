"""GPU parity: W8A8 contraction (skinny GEMV and LDS-tiled MFMA GEMM), the
dequant epilogue and the whole rotated linear.  Gates: int32 accumulators and
int8 codes bit-exact; dequantized fp32 within rel-L2 1e-3 (in fact equal)."""
import numpy as np
import pytest

import workload

pytestmark = pytest.mark.gpu


def rand_codes(seed, shape):
    return np.random.default_rng(seed).integers(-127, 128, shape).astype(np.int8)


def gpu_gemm_i32(mi, dev, qx, qw):
    mark = dev.mark()
    dqx, dqw = dev.upload(qx), dev.upload(qw)
    dacc = dev.empty((qx.shape[0], qw.shape[0]), np.int32)
    mi.gemm_i32(dqx, dqw, dacc)
    acc = dev.download(dacc)
    dev.reset_to(mark)
    return acc


@pytest.mark.parametrize("M,N,K", [
    (1, 64, 128), (1, 6144, 4096), (4, 4096, 14336), (16, 256, 4096), (13, 48, 1024),
    (17, 64, 768), (32, 4096, 4096), (33, 128, 2048), (48, 160, 256), (64, 512, 1408),
    (2, 96, 9216), (3, 80, 11264),    # K that the register-resident GEMV cannot split: the LDS-staged one
    # 5 to 16 tokens with N = 8 * 256 * P rows: the ring kernel with the rows dealt to the compute units in 8-row
    # blocks, P = 3, 5, 7 as two workgroups of unequal size per unit, P = 10, 12, 14 as two equal ones
    (16, 6144, 4096), (5, 6144, 1024), (16, 10240, 1024), (9, 14336, 2048), (16, 14336, 4096),
    (16, 20480, 1024), (12, 24576, 1024), (16, 28672, 4096), (7, 28672, 1024),
])
def test_skinny_accumulators_bit_exact(mi, dev, orc, M, N, K):
    qx, qw = rand_codes(M * 7 + N, (M, K)), rand_codes(K + 1, (N, K))
    assert np.array_equal(gpu_gemm_i32(mi, dev, qx, qw), orc.gemm_i8_i32(qx, qw))


@pytest.mark.parametrize("M,N,K", [
    (65, 256, 128), (128, 128, 256), (256, 256, 1024), (200, 192, 512), (257, 272, 384),
    (512, 448, 768), (300, 1000 // 16 * 16, 640), (2048, 224 * 3, 512), (1024, 6144, 256),
    (4096, 4096, 256),                # the 256 x 256 tile
])
def test_tiled_accumulators_bit_exact(mi, dev, orc, M, N, K):
    qx, qw = rand_codes(M + 3 * N, (M, K)), rand_codes(K + 5, (N, K))
    assert np.array_equal(gpu_gemm_i32(mi, dev, qx, qw), orc.gemm_i8_i32(qx, qw))


@pytest.mark.parametrize("M,N,K", [
    # whole 256 x 192 and 128 x 256 tiles, one per compute unit: the kernel with two waves per SIMD.  K of 1 to 5
    # stages walks every branch of its prologue and of its last stages.
    (2048, 6144, 128), (2048, 6144, 256), (2048, 6144, 384), (2048, 6144, 512), (2048, 6144, 640),
    (2048, 4096, 128), (2048, 4096, 256), (2048, 4096, 384), (2048, 4096, 896),
])
def test_paired_wave_kernel_bit_exact(mi, dev, orc, M, N, K):
    """Every accumulator, then the dequantized form of the same product (fp32, scale by scale as the oracle does)."""
    qx, qw = rand_codes(M + N + K, (M, K)), rand_codes(K + 9, (N, K))
    want = orc.gemm_i8_i32(qx, qw)
    assert np.array_equal(gpu_gemm_i32(mi, dev, qx, qw), want)
    g = np.random.default_rng(K)
    sx = g.uniform(0.01, 1, M).astype(np.float32)
    sw = g.uniform(0.001, 0.1, N).astype(np.float32)
    mark = dev.mark()
    dy = dev.empty((M, N), np.float32)
    mi.check(mi.lib.mi_w8a8_gemm_dequant_f32(dev.upload(qx).ptr, dev.upload(sx).ptr, dev.upload(qw).ptr,
                                             dev.upload(sw).ptr, dy.ptr, M, N, K, None))
    dev.sync()
    y = dev.download(dy)
    dev.reset_to(mark)
    assert np.array_equal(y, orc.dequant(want, sx, sw))


def test_random_skinny_shapes_bit_exact(mi, dev, orc):
    """Seeded random shapes over every skinny path (1 to 64 tokens, K of 1 to 39 stages, N any multiple of 16 or a
    multiple of 2048, which takes the evenly dealt ring kernels): exact against the oracle."""
    rng = np.random.default_rng(7)
    for _ in range(60):
        M, K = int(rng.integers(1, 65)), int(rng.integers(1, 40)) * 128
        N = int(rng.choice([int(rng.integers(1, 300)) * 16, 2048 * int(rng.integers(1, 15))]))
        qx = rng.integers(-127, 128, (M, K)).astype(np.int8)
        qw = rng.integers(-127, 128, (N, K)).astype(np.int8)
        assert np.array_equal(gpu_gemm_i32(mi, dev, qx, qw), orc.gemm_i8_i32(qx, qw)), (M, N, K)


def test_extreme_codes_do_not_overflow(mi, dev):
    K = 14336
    qx = np.full((80, K), 127, np.int8)
    qx[1::2] = -127
    qw = np.full((32, K), 127, np.int8)
    acc = gpu_gemm_i32(mi, dev, qx, qw)
    assert np.all(acc[0::2] == 127 * 127 * K) and np.all(acc[1::2] == -127 * 127 * K)
    acc = gpu_gemm_i32(mi, dev, qx[:16], qw)
    assert np.all(acc[0::2] == 127 * 127 * K) and np.all(acc[1::2] == -127 * 127 * K)


def test_dequant_kernel_matches_closed_form(mi, dev, orc):
    g = np.random.default_rng(3)
    acc = g.integers(-2 ** 27, 2 ** 27, (33, 80)).astype(np.int32)
    sx = g.uniform(0.01, 1, 33).astype(np.float32)
    sw = g.uniform(0.001, 0.1, 80).astype(np.float32)
    mark = dev.mark()
    dy = dev.empty(acc.shape, np.float32)
    mi.dequant(dev.upload(acc), dev.upload(sx), dev.upload(sw), dy)
    y = dev.download(dy)
    dev.reset_to(mark)
    assert np.array_equal(y, orc.dequant(acc, sx, sw))


@pytest.mark.parametrize("M,N,K", [(32, 4096, 4096), (1, 512, 4096), (16, 256, 14336), (130, 320, 1024),
                                   # one token, K <= 4096: the kernel with the quantizer inside; the rest: two kernels
                                   (1, 6144, 4096), (1, 272, 2048), (4, 6144, 4096), (2, 1024, 14336), (1, 4096, 14336)])
def test_whole_linear(mi, dev, orc, M, N, K):
    """cfg0 is the first case: x [32,4096] with outlier channels, W [4096,4096]."""
    x = workload.activations(11, M, K)
    w = workload.weights(12, N, K)
    mark = dev.mark()
    dw = dev.upload(w)
    dqw, dsw = dev.empty((N, K), np.int8), dev.empty(N, np.float32)
    mi.fwht_quant(dw, dqw, dsw, 128)                       # weight prep on the GPU
    qw, sw = dev.download(dqw), dev.download(dsw)
    qwo, swo = orc.rotate_quant_rows(w, 128)
    assert np.array_equal(qw, qwo) and np.array_equal(sw, swo)
    ws = dev.empty(mi.lib.mi_w8a8_linear_workspace_bytes(M, N, K), np.uint8)
    dy = dev.empty((M, N), np.float32)
    mi.linear(dev.upload(x), dqw, dsw, dy, 128, ws)
    y = dev.download(dy)
    qx = dev.download(ws.offset(0, (M, K), np.int8))
    dev.reset_to(mark)
    yo, qxo, sxo, acco = orc.w8a8_linear(x, qwo, swo, 128)
    assert np.array_equal(qx, qxo)
    rel = np.linalg.norm(y.astype(np.float64) - yo) / np.linalg.norm(yo.astype(np.float64))
    assert rel <= 1e-3            # the stated gate
    assert np.array_equal(y, yo)  # and in fact identical: same IEEE operations in the same order


@pytest.mark.parametrize("name,K,N", workload.PROJECTIONS)
@pytest.mark.parametrize("M", [1, 4, 16, 2048])
def test_full_size_projections(mi, dev, orc, name, K, N, M):
    """cfg1 / cfg3 shapes: sampled rows against the oracle plus a linearity
    checksum over every row: sum_n acc[m,n] == qx[m,:] . (sum_n qw[n,:])."""
    qx, qw = rand_codes(31 + M, (M, K)), rand_codes(32 + N, (N, K))
    acc = gpu_gemm_i32(mi, dev, qx, qw)
    colsum = qw.astype(np.int64).sum(axis=0)
    assert np.array_equal(acc.astype(np.int64).sum(axis=1), qx.astype(np.int64) @ colsum)
    rowsum = qx.astype(np.int64).sum(axis=0)
    assert np.array_equal(acc.astype(np.int64).sum(axis=0), qw.astype(np.int64) @ rowsum)
    rows = sorted(set([0, M - 1] + list(np.random.default_rng(M).integers(0, M, 6))))
    assert np.array_equal(acc[rows], orc.gemm_i8_i32(qx[rows], qw))


@pytest.mark.parametrize("name,K,N", [workload.PROJECTIONS[0], workload.PROJECTIONS[3]])
def test_whole_prefill_linear_end_to_end(mi, dev, orc, name, K, N):
    """cfg3, one projection per K: the whole mi_w8a8_linear_f32 at M = 2048 (rotate + quantize, tiled GEMM, dequant)
    against the oracle's linear on sampled rows (the oracle quantizes a row on its own, so a row of y depends on
    that row of x alone), and the activation codes of every row."""
    M = workload.PREFILL_M
    x = workload.activations(21, M, K)
    w = workload.weights(22, N, K)
    mark = dev.mark()
    dqw, dsw = dev.empty((N, K), np.int8), dev.empty(N, np.float32)
    keep = dev.mark()
    mi.fwht_quant(dev.upload(w), dqw, dsw, 128)
    dev.sync()
    dev.reset_to(keep)
    ws = dev.empty(mi.lib.mi_w8a8_linear_workspace_bytes(M, N, K), np.uint8)
    dy = dev.empty((M, N), np.float32)
    mi.linear(dev.upload(x), dqw, dsw, dy, 128, ws)
    y = dev.download(dy)
    qx = dev.download(ws.offset(0, (M, K), np.int8))
    qw, sw = dev.download(dqw), dev.download(dsw)
    dev.reset_to(mark)
    assert np.array_equal(qx, orc.rotate_quant_rows(x, 128)[0])
    rows = sorted(set([0, 255, 256, M - 1] + list(np.random.default_rng(K).integers(0, M, 8))))
    yo = orc.w8a8_linear(x[rows], qw, sw, 128)[0]
    assert np.linalg.norm(y[rows].astype(np.float64) - yo) <= 1e-3 * np.linalg.norm(yo.astype(np.float64))
    assert np.array_equal(y[rows], yo)
    assert np.all(np.isfinite(y))


def test_argument_errors(mi, dev):
    lib = mi.lib
    mark = dev.mark()
    b = dev.empty(1 << 16, np.int8)
    assert lib.mi_w8a8_gemm_i32(b.ptr, b.ptr, b.ptr, 4, 16, 100, None) == mi.EINVAL     # K % 128
    assert lib.mi_w8a8_gemm_i32(b.ptr, b.ptr, b.ptr, 4, 20, 128, None) == mi.EINVAL     # N % 16
    assert lib.mi_w8a8_gemm_i32(b.ptr, b.ptr + 8, b.ptr, 4, 16, 128, None) == mi.EINVAL  # alignment
    assert lib.mi_w8a8_gemm_i32(b.ptr, b.ptr, b.ptr, 4, 16, 133248, None) == mi.ERANGE  # int32 bound
    assert lib.mi_w8a8_gemm_i32(b.ptr, b.ptr, b.ptr, 0, 16, 128, None) == mi.OK
    assert lib.mi_w8a8_linear_f32(b.ptr, b.ptr, b.ptr, b.ptr, 4, 16, 128, 128, b.ptr, 16, None) == mi.ENOSPC
    dev.reset_to(mark)
