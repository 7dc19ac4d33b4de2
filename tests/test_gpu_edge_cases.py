"""Empty batches, ragged sizes next to the tile edges and out-of-range sizes at the C ABI: a call with nothing to do
returns MI_OK and touches no output, a ragged call equals the oracle bit for bit, a size past a documented limit is
refused with its error code before anything is launched."""
import numpy as np
import pytest

import workload

pytestmark = pytest.mark.gpu

POISON = np.float32(-12345.5)


def test_empty_batches_do_nothing(mi, dev):
    lib = mi.lib
    mark = dev.mark()
    K, N, H, I, E, topk = 256, 64, 256, 256, 16, 2
    x = dev.upload(np.zeros((1, K), np.float32))
    q, sc = dev.upload(np.full((1, K), 7, np.int8)), dev.upload(np.full(1, POISON, np.float32))
    assert lib.mi_fwht_quant_f32_i8(x.ptr, q.ptr, sc.ptr, 0, K, 128, None) == 0
    qw, sw = dev.upload(np.ones((N, K), np.int8)), dev.upload(np.ones(N, np.float32))
    y = dev.upload(np.full((1, N), POISON, np.float32))
    ws = dev.empty(max(256, lib.mi_w8a8_linear_workspace_bytes(1, N, K)), np.uint8)
    assert lib.mi_w8a8_linear_f32(x.ptr, qw.ptr, sw.ptr, y.ptr, 0, N, K, 128, ws.ptr, ws.nbytes, None) == 0
    assert lib.mi_w8a8_gemm_dequant_f32(q.ptr, sc.ptr, qw.ptr, sw.ptr, y.ptr, 0, N, K, None) == 0
    acc = dev.upload(np.full((1, N), 77, np.int32))
    assert lib.mi_w8a8_gemm_i32(q.ptr, qw.ptr, acc.ptr, 0, N, K, None) == 0
    # an MoE layer over no tokens
    wr = dev.upload(workload.weights(1, E, H))
    wg = dev.upload(np.ones((E, I, H), np.int8)); wd = dev.upload(np.ones((E, H, I), np.int8))
    sg, sd = dev.upload(np.ones((E, I), np.float32)), dev.upload(np.ones((E, H), np.float32))
    ym = dev.upload(np.full((1, H), POISON, np.float32))
    mws = dev.empty(max(256, lib.mi_moe_layer_workspace_bytes(0, H, I, E, topk)), np.uint8)
    assert lib.mi_moe_layer(x.ptr, wr.ptr, wg.ptr, sg.ptr, wg.ptr, sg.ptr, wd.ptr, sd.ptr, ym.ptr, 0, H, I, E, topk,
                            mws.ptr, mws.nbytes, None) == 0
    idx, w = dev.upload(np.zeros((1, topk), np.int32)), dev.upload(np.zeros((1, topk), np.float32))
    assert lib.mi_moe_ffn(x.ptr, idx.ptr, w.ptr, wg.ptr, sg.ptr, wg.ptr, sg.ptr, wd.ptr, sd.ptr, ym.ptr, 0, H, I, E,
                          topk, mws.ptr, mws.nbytes, None) == 0
    dev.sync()
    assert np.all(dev.download(q) == 7) and dev.download(sc)[0] == POISON
    assert np.all(dev.download(y) == POISON) and np.all(dev.download(acc) == 77)
    assert np.all(dev.download(ym) == POISON)
    dev.reset_to(mark)


@pytest.mark.parametrize("M,N,K", [(1, 16, 128), (3, 17 * 16, 384), (63, 48, 640), (65, 208, 256), (257, 272, 128),
                                   (255, 193 * 16, 384)])
def test_ragged_linear_next_to_the_tile_edges(mi, dev, orc, M, N, K):
    """Row and channel counts one off the kernels' tile sizes (16-row MFMA groups, 64-token skinny limit, 128 / 256
    wide prefill tiles), K of one to five rotation blocks: the whole linear against the oracle."""
    mark = dev.mark()
    x, w = workload.activations(900 + M, M, K), workload.weights(901 + N, N, K)
    qw, sw = orc.rotate_quant_rows(w, 128)
    dqw, dsw = dev.upload(qw), dev.upload(sw)
    ws = dev.empty(mi.lib.mi_w8a8_linear_workspace_bytes(M, N, K), np.uint8)
    dy = dev.empty((M, N), np.float32)
    mi.linear(dev.upload(x), dqw, dsw, dy, 128, ws)
    yo, qxo, _, acco = orc.w8a8_linear(x, qw, sw, 128)
    assert np.array_equal(dev.download(ws.offset(0, (M, K), np.int8)), qxo)
    assert np.array_equal(dev.download(dy), yo)
    dacc = dev.empty((M, N), np.int32)
    mi.check(mi.lib.mi_w8a8_gemm_i32(ws.ptr, dqw.ptr, dacc.ptr, M, N, K, None))
    assert np.array_equal(dev.download(dacc), acco)
    dev.reset_to(mark)


def test_sizes_past_the_limits_are_refused(mi, dev):
    lib = mi.lib
    mark = dev.mark()
    b = dev.empty(1 << 16, np.uint8)
    p = b.ptr
    EINVAL, ERANGE = -22, -34
    # rotation block that does not divide K, K that is no multiple of 128
    assert lib.mi_fwht_quant_f32_i8(p, p, p, 4, 192, 128, None) == EINVAL
    assert lib.mi_w8a8_gemm_i32(p, p, p, 4, 16, 24, None) == EINVAL
    assert lib.mi_w8a8_gemm_i32(p, p, p, 4, 40, 128, None) == EINVAL   # channel counts come in sixteens
    # MoE: more picks than experts, inner size that is no multiple of the 256 block, top-k above the compiled maximum
    assert lib.mi_moe_ffn_workspace_bytes(8, 256, 256, 4, 8) == EINVAL
    assert lib.mi_moe_ffn_workspace_bytes(8, 256, 192, 16, 2) == EINVAL
    assert lib.mi_moe_ffn_workspace_bytes(8, 256, 256, 64, 9) == EINVAL
    # attention: more than four query heads per KV head, a head size other than 128
    assert lib.mi_gqa_decode_workspace_bytes(1, 40, 8, 128, 64) < 0
    assert lib.mi_gqa_decode_workspace_bytes(1, 8, 8, 64, 64) < 0
    # the no-allocation linear beyond its static scratch
    rows = lib.mi_w8a8_linear_noalloc_max_rows()
    assert lib.mi_w8a8_linear_f32_noalloc(p, p, p, p, rows + 1, 16, 128, 128, None) == ERANGE
    dev.reset_to(mark)
