"""The rotated W8A8 linear through the entry point that allocates nothing (its activation codes and scales live
in a static device array): same bits as mi_w8a8_linear_f32 with a caller workspace, on two calls in a row, the
second with a smaller input, so that what the first call left in the array is shown not to leak into the second.
Collected last on purpose (file name): a failure here must not hide the other GPU tests."""
import numpy as np
import pytest

import workload

pytestmark = pytest.mark.gpu


def _both(mi, dev, x, dqw, dsw, block):
    """y from the workspace entry point and y from the no-alloc one, for one input."""
    M, K = x.shape
    N = dqw.shape[0]
    mark = dev.mark()
    dx = dev.upload(x)
    ws = dev.empty(mi.lib.mi_w8a8_linear_workspace_bytes(M, N, K), np.uint8)
    y_ref, y_new = dev.empty((M, N), np.float32), dev.empty((M, N), np.float32)
    mi.check(mi.lib.mi_fill_u32(y_new.ptr, 0x7fc00000, M * N, None), "mi_fill_u32")   # NaN: every element must be written
    mi.linear(dx, dqw, dsw, y_ref, block, ws)
    mi.check(mi.lib.mi_w8a8_linear_f32_noalloc(dx.ptr, dqw.ptr, dsw.ptr, y_new.ptr, M, N, K, block, None),
             "mi_w8a8_linear_f32_noalloc")
    a, b = dev.download(y_ref), dev.download(y_new)
    dev.reset_to(mark)
    return a, b


@pytest.mark.parametrize("shapes", [
    # (M, N, K) of the first call, then of the smaller second call
    ((32, 4096, 4096), (16, 512, 1024)),       # ring kernel, then a smaller ring problem
    ((256, 768, 2048), (1, 768, 2048)),        # LDS-tiled GEMM, then the one-kernel decode linear
    ((4, 256, 14336), (3, 256, 1024)),         # register GEMV on a long row, then a short one
])
def test_noalloc_linear_equals_workspace_linear_twice(mi, dev, orc, shapes):
    for call, (M, N, K) in enumerate(shapes):
        w = workload.weights(100 + N + K, N, K)
        mark = dev.mark()
        dqw, dsw = dev.empty((N, K), np.int8), dev.empty(N, np.float32)
        keep = dev.mark()
        mi.fwht_quant(dev.upload(w), dqw, dsw, 128)
        dev.sync()
        dev.reset_to(keep)
        x = workload.activations(7 + call + M, M, K)
        y_ref, y_new = _both(mi, dev, x, dqw, dsw, 128)
        assert not np.isnan(y_new).any()
        assert np.array_equal(y_ref, y_new), "call %d (M=%d N=%d K=%d) differs" % (call, M, N, K)
        if M * N * K <= 32 * 4096 * 4096:
            qw, sw = dev.download(dqw), dev.download(dsw)
            yo = orc.w8a8_linear(x, qw, sw, 128)[0]
            assert np.linalg.norm(y_new - yo) <= 1e-3 * np.linalg.norm(yo)
        dev.reset_to(mark)


def test_noalloc_limits_are_refused(mi, dev):
    lib = mi.lib
    rows, codes = lib.mi_w8a8_linear_noalloc_max_rows(), lib.mi_w8a8_linear_noalloc_max_codes()
    assert rows == 8192 and codes == 8 << 20
    mark = dev.mark()
    buf = dev.empty(4096, np.uint8)   # never dereferenced: the size check comes first
    p = buf.ptr
    assert lib.mi_w8a8_linear_f32_noalloc(p, p, p, p, rows + 1, 16, 128, 128, None) == mi.ERANGE
    assert lib.mi_w8a8_linear_f32_noalloc(p, p, p, p, 2048, 16, 4096 + 128, 128, None) == mi.ERANGE
    assert lib.mi_w8a8_linear_f32_noalloc(p, p, p, p, 1, 16, codes + 128, 128, None) == mi.ERANGE
    assert lib.mi_w8a8_linear_f32_noalloc(None, p, p, p, 1, 16, 128, 128, None) == mi.EINVAL
    dev.reset_to(mark)
