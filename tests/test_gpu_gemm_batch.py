"""GPU parity: several W8A8 contractions in one launch (mi_gemm_batch_*), the kernel whose workgroups walk a list of
256 x 256 tiles.  Gates: int32 accumulators bit-exact against the oracle; the dequantized form equal to the
oracle's fp32 operations; both equal, bit for bit, to the single-problem entry points."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def rand_codes(seed, shape):
    return np.random.default_rng(seed).integers(-127, 128, shape).astype(np.int8)


def make_ops(dev, shapes, seed, dtype):
    """Upload codes (and scales) for every problem; returns the device operand tuples and the host arrays."""
    ops, host = [], []
    for i, (M, N, K) in enumerate(shapes):
        qx, qw = rand_codes(seed + 11 * i, (M, K)), rand_codes(seed + 11 * i + 5, (N, K))
        g = np.random.default_rng(seed + i)
        sx = g.uniform(0.01, 1, M).astype(np.float32)
        sw = g.uniform(0.001, 0.1, N).astype(np.float32)
        out = dev.empty((M, N), dtype)
        ops.append((dev.upload(qx), dev.upload(sx), dev.upload(qw), dev.upload(sw), out))
        host.append((qx, sx, qw, sw))
    return ops, host


# K of 3 to 7 stages (short tiles: the stores of the tile before them are still in flight when they end) and of 24, 25
# and 32; shapes that are no multiple of the tile exercise the tiles that are moved inwards (rows: 300 = 256 + 44,
# columns: 272 = 256 + 16, 1168 = 4 * 256 + 144); several tiles per workgroup exercise the load
# stream across tile boundaries, the scales that change registers' contents between tiles and the clearing of the
# accumulators; mixed K in one batch exercises a cursor that changes its stride between tiles.
@pytest.mark.parametrize("shapes", [
    [(256, 256, 384)],
    [(256, 256, 512)],
    [(300, 272, 640)],
    [(2048, 6144, 384)],
    [(2048, 6144, 896)],
    [(2048, 14336, 384)],
    [(4096, 4096, 512)],
    [(2048, 4608, 3072)],
    [(2048, 6144, 3200)],
    [(512, 384, 896), (256, 272, 384)],
    [(2048, 6144, 384), (2048, 4096, 4096), (264, 14336, 512)],
    [(1024, 1168, 768)] * 8,
])
def test_batch_accumulators_bit_exact(mi, dev, orc, shapes):
    mark = dev.mark()
    batch = mi.GemmBatch(dev, shapes)
    ops, host = make_ops(dev, shapes, 1000 + len(shapes) + shapes[0][2], np.int32)
    for o in ops:   # poison: every element must be written
        mi.check(mi.lib.mi_fill_u32(o[4].ptr, 0x7F7F7F7F, o[4].nbytes // 4, None))
    batch.run_i32([(qx, None, qw, None, out) for qx, _, qw, _, out in ops])
    dev.sync()
    for (M, N, K), o, (qx, sx, qw, sw) in zip(shapes, ops, host):
        assert np.array_equal(dev.download(o[4]), orc.gemm_i8_i32(qx, qw)), (M, N, K)
    batch.destroy()
    dev.reset_to(mark)


@pytest.mark.parametrize("shapes", [
    [(256, 256, 384)],
    [(300, 272, 512)],
    [(2048, 6144, 384), (520, 4096, 1024)],
    [(2048, 6144, 4096)],
])
def test_batch_dequant_equals_the_oracle_and_the_single_call(mi, dev, orc, shapes):
    mark = dev.mark()
    batch = mi.GemmBatch(dev, shapes)
    ops, host = make_ops(dev, shapes, 77, np.float32)
    batch.run_f32(ops)
    batch.run_f32(ops)   # a second run on the same batch: nothing of the first is left behind
    dev.sync()
    for (M, N, K), (dqx, dsx, dqw, dsw, dy), (qx, sx, qw, sw) in zip(shapes, ops, host):
        y = dev.download(dy)
        assert np.array_equal(y, orc.dequant(orc.gemm_i8_i32(qx, qw), sx, sw)), (M, N, K)
        dy1 = dev.empty((M, N), np.float32)
        mi.check(mi.lib.mi_w8a8_gemm_dequant_f32(dqx.ptr, dsx.ptr, dqw.ptr, dsw.ptr, dy1.ptr, M, N, K, None))
        dev.sync()
        assert np.array_equal(y, dev.download(dy1)), (M, N, K)
    batch.destroy()
    dev.reset_to(mark)


def test_batch_full_size_projections(mi, dev, orc):
    """The four M = 2048 projections of the prefill configuration as one launch: checksums over every element
    against the single-problem kernels, sampled rows against the oracle."""
    shapes = [(2048, 6144, 4096), (2048, 14336, 4096), (2048, 14336, 4096), (2048, 4096, 14336)]
    mark = dev.mark()
    batch = mi.GemmBatch(dev, shapes)
    ops, host = make_ops(dev, shapes, 4242, np.int32)
    batch.run_i32([(qx, None, qw, None, out) for qx, _, qw, _, out in ops])
    dev.sync()
    rows = np.array([0, 1, 255, 256, 1023, 1791, 1792, 2047])
    for (M, N, K), (dqx, _, dqw, _, dacc), (qx, sx, qw, sw) in zip(shapes, ops, host):
        acc = dev.download(dacc)
        assert np.array_equal(acc[rows], orc.gemm_i8_i32(qx[rows], qw)), (M, N, K)
        m2 = dev.mark()
        dref = dev.empty((M, N), np.int32)
        mi.gemm_i32(dqx, dqw, dref)
        dev.sync()
        assert np.array_equal(acc, dev.download(dref)), (M, N, K)
        dev.reset_to(m2)
    batch.destroy()
    dev.reset_to(mark)


def test_batch_rejects_what_it_cannot_run(mi, dev):
    import ctypes as C
    i64 = C.c_int64

    def plan_bytes(shapes):
        arr = (i64 * (3 * len(shapes)))(*[v for s in shapes for v in s])
        return mi.lib.mi_gemm_batch_plan_bytes(arr, len(shapes))

    assert plan_bytes([(255, 256, 384)]) == mi.EINVAL      # fewer rows than a tile
    assert plan_bytes([(256, 240, 384)]) == mi.EINVAL      # fewer columns than a tile
    assert plan_bytes([(256, 264, 384)]) == mi.EINVAL      # N % 16
    assert plan_bytes([(256, 256, 448)]) == mi.EINVAL      # K % 128
    assert plan_bytes([(256, 256, 256)]) == mi.EINVAL      # fewer than three K stages
    assert plan_bytes([(256, 256, 384)] * 9) == mi.EINVAL  # more than eight problems
    assert plan_bytes([(256, 256, 1 << 18)]) == mi.ERANGE  # the int32 accumulator could overflow
    assert plan_bytes([(256, 256, 384)]) > 0
    mark = dev.mark()
    batch = mi.GemmBatch(dev, [(256, 256, 384)])
    qx, qw, out = dev.empty((256, 512), np.int8), dev.empty((256, 512), np.int8), dev.empty((256, 256), np.int32)
    with pytest.raises(mi.MiError) as e:   # K differs from the batch's
        batch.run_i32([(qx, None, qw, None, out)])
    assert e.value.status == mi.EINVAL
    batch.destroy()
    dev.reset_to(mark)


def test_random_batches_equal_the_single_problem_kernels(mi, dev):
    """Seeded random batches (1 to 4 problems, ragged M and N, 3 to 19 K stages, mixed K in one batch): every
    dequantized output equals, bit for bit, what the single-problem entry point writes for the same operands."""
    rng = np.random.default_rng(20251125)
    for _ in range(12):
        shapes = [(int(rng.integers(256, 1200)), max(256, int(rng.integers(16, 90)) * 16), int(rng.integers(3, 20)) * 128)
                  for _ in range(int(rng.integers(1, 5)))]
        mark = dev.mark()
        ops, refs = [], []
        for M, N, K in shapes:
            qx = dev.upload(rng.integers(-127, 128, (M, K)).astype(np.int8))
            qw = dev.upload(rng.integers(-127, 128, (N, K)).astype(np.int8))
            sx = dev.upload(rng.uniform(0.01, 1, M).astype(np.float32))
            sw = dev.upload(rng.uniform(0.001, 0.1, N).astype(np.float32))
            y, ref = dev.empty((M, N), np.float32), dev.empty((M, N), np.float32)
            mi.check(mi.lib.mi_fill_u32(y.ptr, 0x7F7F7F7F, y.nbytes // 4, None))   # poison: every element must be written
            mi.check(mi.lib.mi_w8a8_gemm_dequant_f32(qx.ptr, sx.ptr, qw.ptr, sw.ptr, ref.ptr, M, N, K, None))
            ops.append((qx, sx, qw, sw, y))
            refs.append(ref)
        batch = mi.GemmBatch(dev, shapes)
        batch.run_f32(ops)
        dev.sync()
        for s, o, r in zip(shapes, ops, refs):
            assert np.array_equal(dev.download(o[4]), dev.download(r)), (shapes, s)
        batch.destroy()
        dev.reset_to(mark)
