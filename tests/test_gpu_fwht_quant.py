"""GPU parity: fused block-Hadamard + int8 row quantizer against the CPU
restatement.  Gate: codes and scales bit-exact (integer / IEEE fp32 work)."""
import numpy as np
import pytest

import workload

pytestmark = pytest.mark.gpu


def run_quant(mi, dev, x, block):
    mark = dev.mark()
    dx = dev.upload(x)
    dq = dev.empty(x.shape, np.int8)
    ds = dev.empty(x.shape[0], np.float32)
    mi.fwht_quant(dx, dq, ds, block)
    q, s = dev.download(dq), dev.download(ds)
    dev.reset_to(mark)
    return q, s


@pytest.mark.parametrize("M,K,block", [
    (32, 4096, 128),      # cfg0 activations
    (16, 14336, 128),     # decode down-projection input (7 chunks per thread)
    (1, 4096, 128),
    (5, 2048, 128),       # MoE hidden
    (37, 768, 256),       # MoE inner dim, 3 blocks of 256
    (1501, 768, 256),     # many short rows: the wave-per-row kernel (ragged last workgroup)
    (1024, 2048, 128),    # wave-per-row, four chunks per lane
    (1030, 256, 256),     # wave-per-row, half of the lanes idle
    (64, 128, 128),       # attention heads / KV rows: one block per row
    (1000, 128, 128),     # ragged count of small rows
    (9, 256, 256),
    (3, 256, 128),
    (2, 6144, 128),       # 3 chunks per thread -> padded to 4
    (2, 32768, 128),      # largest supported row
])
def test_codes_and_scales_bit_exact(mi, dev, orc, M, K, block):
    x = workload.activations(1234 + M + K, M, K)
    q, s = run_quant(mi, dev, x, block)
    qo, so = orc.rotate_quant_rows(x, block)
    assert np.array_equal(s, so)
    assert np.array_equal(q, qo)

@pytest.mark.parametrize("shapes,block", [
    ([(33, 4096), (17, 4096), (9, 14336)], 128),            # the prefill step's three inputs, small
    ([(5, 2048), (3, 32768), (2, 6144), (4, 8192)], 128),   # 1, 16, 3 -> 4 and 4 chunks per thread in one launch
    ([(7, 4096), (6, 2048)], 256),
    ([(8, 4096), (5, 768)], 256),                           # a short-row set: the call takes one launch per set
    ([(40, 2048)] * 8, 128),                                # the most sets a call takes
])
def test_batched_quantizer_is_the_single_calls(mi, dev, orc, shapes, block):
    """mi_fwht_quant_batch_f32_i8: every set's codes and scales are the oracle's (and so those of separate calls);
    the rows of one set do not leak into the next (poisoned outputs, sets of different K side by side)."""
    mark = dev.mark()
    xs = [workload.activations(77 + i, M, K, stream=K + i) for i, (M, K) in enumerate(shapes)]
    sets = []
    for x in xs:
        q, s = dev.empty(x.shape, np.int8), dev.empty(x.shape[0], np.float32)
        mi.check(mi.lib.mi_fill_u32(q.ptr, 0x7F7F7F7F, q.nbytes // 4, None))
        sets.append((dev.upload(x), q, s))
    mi.fwht_quant_batch(sets, block)
    for x, (_, dq, ds) in zip(xs, sets):
        qo, so = orc.rotate_quant_rows(x, block)
        assert np.array_equal(dev.download(ds), so)
        assert np.array_equal(dev.download(dq), qo)
    dev.reset_to(mark)


def test_batched_quantizer_full_size_and_errors(mi, dev, orc):
    """The three inputs of the prefill configuration in one launch against three launches, bit for bit; argument
    errors as the single call reports them."""
    mark = dev.mark()
    shapes = [(2048, 4096), (2048, 4096), (2048, 14336)]
    xs = [dev.upload(workload.activations(5, M, K, stream=i)) for i, (M, K) in enumerate(shapes)]
    one = [(x, dev.empty(x.shape, np.int8), dev.empty(x.shape[0], np.float32)) for x in xs]
    three = [(x, dev.empty(x.shape, np.int8), dev.empty(x.shape[0], np.float32)) for x in xs]
    mi.fwht_quant_batch(one, 128)
    for x, q, s in three:
        mi.fwht_quant(x, q, s, 128)
    for (_, q1, s1), (_, q3, s3) in zip(one, three):
        assert np.array_equal(dev.download(q1), dev.download(q3)) and np.array_equal(dev.download(s1), dev.download(s3))
    arr = (mi.QuantRows * 9)()
    assert mi.lib.mi_fwht_quant_batch_f32_i8(arr, 9, 128, None) == mi.EINVAL      # more than eight sets
    assert mi.lib.mi_fwht_quant_batch_f32_i8(arr, 0, 128, None) == mi.EINVAL
    assert mi.lib.mi_fwht_quant_batch_f32_i8(None, 1, 128, None) == mi.EINVAL
    arr[0].x, arr[0].q, arr[0].scale, arr[0].M, arr[0].K = one[0][0].ptr, one[0][1].ptr, one[0][2].ptr, 4, 4000
    assert mi.lib.mi_fwht_quant_batch_f32_i8(arr, 1, 128, None) == mi.EINVAL      # K % block
    dev.reset_to(mark)


def test_weight_prep_bit_exact(mi, dev, orc):
    w = workload.weights(7, 1024, 4096)
    q, s = run_quant(mi, dev, w, 128)
    qo, so = orc.rotate_quant_rows(w, 128)
    assert np.array_equal(s, so) and np.array_equal(q, qo)


def test_zero_rows_ties_and_extremes(mi, dev, orc):
    x = workload.activations(5, 8, 256)
    x[2] = 0.0                        # all-zero row: scale 1, codes 0
    x[3] = 0.0
    x[3, 17] = 3.0e38                 # one huge value
    x[4] = 1.0e-30                    # tiny but non-zero
    x[5] = np.arange(256, dtype=np.float32) - 128.0   # integers: exact halves after scaling
    q, s = run_quant(mi, dev, x, 128)
    qo, so = orc.rotate_quant_rows(x, 128)
    assert s[2] == 1.0 and not q[2].any()
    assert np.array_equal(s, so) and np.array_equal(q, qo)


@pytest.mark.parametrize("M,K,block", [(9, 512, 128), (1030, 256, 128), (40, 128, 128), (5, 768, 256)])
def test_non_finite_rows_follow_the_oracle(mi, dev, orc, M, K, block):
    """NaN and +-Inf inputs (which the rotation spreads over their block) quantize the same way on both sides, in
    each of the three kernels (a workgroup per row, a wave per row, 16 lanes per row): nothing is undefined."""
    x = workload.activations(6, M, K)
    x[1, 3] = np.nan
    x[2, K - 1] = np.inf
    x[3, 0], x[3, block // 2] = np.inf, -np.inf
    x[4] = np.nan
    x[M - 1, K // 2] = -np.inf
    with np.errstate(invalid="ignore"):
        q, s = run_quant(mi, dev, x, block)
        qo, so = orc.rotate_quant_rows(x, block)
    assert np.array_equal(q, qo)
    assert np.array_equal(s, so, equal_nan=True)
    assert s[4] == 1.0 and np.all(q[4] == -127)           # a row of NaNs: absmax 0, every product NaN
    assert np.all(q[1, :block] == -127)                    # the NaN's block
    assert np.array_equal(q[0], orc.rotate_quant_rows(x[:1], block)[0][0])


@pytest.mark.parametrize("M,K,block", [(7, 4096, 128), (3, 768, 256), (33, 128, 128), (1027, 512, 256)])
def test_rotation_only_bit_exact_and_in_place(mi, dev, orc, M, K, block):
    x = workload.normal(3, (M, K))
    mark = dev.mark()
    dx = dev.upload(x)
    dout = dev.empty(x.shape, np.float32)
    mi.fwht(dx, dout, block)
    out = dev.download(dout)
    mi.fwht(dx, dx, block)            # aliasing allowed
    inplace = dev.download(dx)
    dev.reset_to(mark)
    want = orc.rotate_rows(x, block)
    assert np.array_equal(out, want) and np.array_equal(inplace, want)


def test_full_size_properties(mi, dev, orc):
    """cfg3-sized activations: spot rows bit-exact, invariants on all rows."""
    M, K = 2048, 14336
    x = workload.activations(99, M, K)
    q, s = run_quant(mi, dev, x, 128)
    rows = [0, 1, 777, 2047]
    qo, so = orc.rotate_quant_rows(x[rows], 128)
    assert np.array_equal(q[rows], qo) and np.array_equal(s[rows], so)
    assert np.all(np.max(np.abs(q.astype(np.int16)), axis=1) == 127)
    # rotation preserves the row norm: sum (q*s)^2 ~= sum x^2 up to quantization noise
    n_in = np.linalg.norm(x.astype(np.float64), axis=1)
    n_out = np.linalg.norm(q.astype(np.float64), axis=1) * s
    assert np.max(np.abs(n_out / n_in - 1)) < 2e-2


def test_argument_errors(mi, dev):
    lib = mi.lib
    mark = dev.mark()
    b = dev.empty(4096, np.float32)
    assert lib.mi_fwht_quant_f32_i8(b.ptr, b.ptr, b.ptr, 1, 100, 128, None) == mi.EINVAL   # K % block
    assert lib.mi_fwht_quant_f32_i8(b.ptr, b.ptr, b.ptr, 1, 192, 64, None) == mi.EINVAL    # block size
    assert lib.mi_fwht_quant_f32_i8(b.ptr, b.ptr, b.ptr, 1, 65536, 128, None) == mi.ERANGE
    assert lib.mi_fwht_quant_f32_i8(b.ptr + 4, b.ptr, b.ptr, 1, 128, 128, None) == mi.EINVAL  # alignment
    assert lib.mi_fwht_quant_f32_i8(b.ptr, b.ptr, b.ptr, 0, 128, 128, None) == mi.OK       # empty input
    dev.reset_to(mark)
