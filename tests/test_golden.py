"""The committed fixture tests/golden/hotpath.npz against (a) the CPU oracle and (b) the HIP library.

The upstream repository holds no vector for this path, so the fixture is the oracle's own output on small
deterministic inputs (tests/golden/gen.py builds them by integer hashing; tests/golden/make_fixtures.py wrote the
expected arrays).  It freezes the oracle's DECISIONS as data: integer results must match bit for bit, results that
pass through expf within the tolerances stated here."""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import gen   # noqa: E402


@pytest.fixture(scope="module")
def gold():
    with np.load(os.path.join(HERE, "golden", "hotpath.npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def layer_inputs():
    R, W, eps, salt = gen.LAYER
    return (gen.bell((R, W), salt), gen.bell((R, W), salt + 1), gen.bell((W,), salt + 2, 0.3) + np.float32(1),
            gen.bell((R, 2 * W), salt + 3, 2.0), eps)


# ---------------------------------------------------------------- the oracle reproduces the fixture (CPU)
def test_oracle_fwht_quant(orc, gold):
    for name, shape, block, salt in gen.FWHT:
        q, s, xr = orc.rotate_quant_rows(gen.fwht_input(shape, salt), block, want_rot=True)
        assert np.array_equal(q, gold["fwht_%s_q" % name]) and np.array_equal(s, gold["fwht_%s_s" % name])
        assert np.array_equal(xr, gold["fwht_%s_rot" % name])
        assert not q[0].any() and s[0] == 1.0                      # the all-zero row
        assert np.abs(q[1:]).max(axis=1).min() == 127              # every other row reaches full scale


def test_oracle_gemm_linear(orc, gold):
    M, N, K, salt = gen.GEMM
    assert np.array_equal(orc.gemm_i8_i32(gen.codes((M, K), salt), gen.codes((N, K), salt + 1)), gold["gemm_acc"])
    M, N, K, b, salt = gen.LINEAR
    qw, sw = orc.rotate_quant_rows(gen.bell((N, K), salt + 1, 0.02), b)
    assert np.array_equal(qw, gold["linear_qw"]) and np.array_equal(sw, gold["linear_sw"])
    y, _, _, acc = orc.w8a8_linear(gen.fwht_input((M, K), salt), qw, sw, b)
    assert np.array_equal(acc, gold["linear_acc"]) and np.array_equal(y, gold["linear_y"])


def test_oracle_attention(orc, gold):
    q, kq, ks, vq, vs = gen.attn_inputs()
    o, qq, sq, dots = orc.gqa_decode(q, kq, ks, vq, vs, out_rotated=False, want_debug=True)
    assert np.array_equal(qq, gold["attn_qq"]) and np.array_equal(sq, gold["attn_sq"])
    assert np.array_equal(dots, gold["attn_dots"])
    assert np.max(np.abs(o - gold["attn_o"])) <= 1e-6              # float64 exp: libm may differ in the last place
    assert np.max(np.abs(orc.gqa_decode(q, kq, ks, vq, vs, out_rotated=True) - gold["attn_o_rot"])) <= 1e-6


def test_oracle_moe(orc, gold):
    T, H, I, E, topk, salt = gen.MOE
    x, wr, wg, sg, wu, su, wd, sd = gen.moe_inputs()
    idx, w, lg = orc.moe_route(x, wr, topk, want_logits=True)
    assert np.array_equal(idx, gold["moe_idx"]) and np.array_equal(lg, gold["moe_logits"])
    assert np.max(np.abs(w - gold["moe_w"])) <= 1e-6
    perm, seg = orc.moe_dispatch(idx, E)
    assert np.array_equal(perm, gold["moe_perm"]) and np.array_equal(seg, gold["moe_seg"])
    y, h, hq, hs, _ = orc.moe_ffn(x, gold["moe_idx"], gold["moe_w"], wg, sg, wu, su, wd, sd, 128, 256, want_debug=True)
    assert np.max(np.abs(h - gold["moe_h"])) <= 1e-6 * max(1.0, float(np.abs(gold["moe_h"]).max()))
    rel = np.linalg.norm(y.astype(np.float64) - gold["moe_y"]) / np.linalg.norm(gold["moe_y"].astype(np.float64))
    assert rel <= 1e-5


def test_oracle_layer_ops(orc, gold):
    x, res, g, gu, eps = layer_inputs()
    h, y = orc.rmsnorm(x, g, eps, residual=res)
    assert np.array_equal(h, gold["rms_h"]) and np.array_equal(y, gold["rms_y"])
    assert np.max(np.abs(orc.swiglu(gu) - gold["swiglu_h"])) <= 1e-6 * float(np.abs(gold["swiglu_h"]).max())
    rows, npos, salt = gen.ROPE
    out = orc.rope_rows(gen.bell((rows, 128), salt), gold["rope_pos"], gold["rope_cos"], gold["rope_sin"])
    assert np.array_equal(out, gold["rope_out"])


# ---------------------------------------------------------------- the HIP library reproduces the fixture (GPU)
@pytest.mark.gpu
def test_gpu_fwht_quant_gemm_linear(mi, dev, gold):
    mark = dev.mark()
    for name, shape, block, salt in gen.FWHT:
        dx = dev.upload(gen.fwht_input(shape, salt))
        dq, ds = dev.empty(shape, np.int8), dev.empty(shape[0], np.float32)
        mi.fwht_quant(dx, dq, ds, block)
        assert np.array_equal(dev.download(dq), gold["fwht_%s_q" % name])
        assert np.array_equal(dev.download(ds), gold["fwht_%s_s" % name])
        drot = dev.empty(shape, np.float32)
        mi.fwht(dx, drot, block)
        assert np.array_equal(dev.download(drot), gold["fwht_%s_rot" % name])
    M, N, K, salt = gen.GEMM
    dacc = dev.empty((M, N), np.int32)
    mi.gemm_i32(dev.upload(gen.codes((M, K), salt)), dev.upload(gen.codes((N, K), salt + 1)), dacc)
    assert np.array_equal(dev.download(dacc), gold["gemm_acc"])
    M, N, K, b, salt = gen.LINEAR
    dw = dev.upload(gen.bell((N, K), salt + 1, 0.02))
    dqw, dsw = dev.empty((N, K), np.int8), dev.empty(N, np.float32)
    mi.fwht_quant(dw, dqw, dsw, b)                                  # weight preparation on the GPU
    assert np.array_equal(dev.download(dqw), gold["linear_qw"]) and np.array_equal(dev.download(dsw), gold["linear_sw"])
    ws = dev.empty(mi.lib.mi_w8a8_linear_workspace_bytes(M, N, K), np.uint8)
    dy = dev.empty((M, N), np.float32)
    mi.linear(dev.upload(gen.fwht_input((M, K), salt)), dqw, dsw, dy, b, ws)
    assert np.array_equal(dev.download(dy), gold["linear_y"])
    dev.reset_to(mark)


@pytest.mark.gpu
def test_gpu_attention(mi, dev, gold):
    mark = dev.mark()
    B, Hq, Hkv, T, _ = gen.ATTN
    q, kq, ks, vq, vs = gen.attn_inputs()
    dq, dkq, dks, dvq, dvs = (dev.upload(a) for a in (q, kq, ks, vq, vs))
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, 128, T), np.uint8)
    do = dev.empty((B, Hq, 128), np.float32)
    dqq, dsq, ddots = dev.empty((B, Hq, 128), np.int8), dev.empty((B, Hq), np.float32), dev.empty((B, Hq, T), np.int32)
    mi.gqa_scores(dq, dkq, dks, dvq, dvs, dqq, dsq, ddots, ws)
    assert np.array_equal(dev.download(dqq), gold["attn_qq"]) and np.array_equal(dev.download(dsq), gold["attn_sq"])
    assert np.array_equal(dev.download(ddots), gold["attn_dots"])
    mi.gqa_decode(dq, dkq, dks, dvq, dvs, do, False, ws)
    assert np.max(np.abs(dev.download(do) - gold["attn_o"])) <= 2e-3          # the gate of the path
    assert np.max(np.abs(dev.download(do) - gold["attn_o"])) <= 2e-5          # what fp32 accumulation gives
    mi.gqa_decode(dq, dkq, dks, dvq, dvs, do, True, ws)
    assert np.max(np.abs(dev.download(do) - gold["attn_o_rot"])) <= 2e-5
    dev.reset_to(mark)


@pytest.mark.gpu
def test_gpu_attention_tiled_layouts(mi, dev, gold):
    """The same fixture through the cache in the matrix-pipe layouts (37 tokens in a cache of 64, junk scales behind
    them): the kernel's own query codes, scales and int32 scores against the committed ones, bit for bit; outputs
    within the gate."""
    mark = dev.mark()
    B, Hq, Hkv, T, _ = gen.ATTN
    T_cap = 64
    q, kq, ks, vq, vs = gen.attn_inputs()
    pad = lambda a, fill: np.concatenate([a, np.full(a.shape[:2] + (T_cap - T,) + a.shape[3:], fill, a.dtype)], axis=2)
    dkq, dvq = dev.upload(pad(kq, 77)), dev.upload(pad(vq, -77))
    dks, dvs = dev.upload(pad(ks, np.nan)), dev.upload(pad(vs, np.nan))
    dkt, dvt = dev.empty((B, Hkv, T_cap, 128), np.int8), dev.empty((B, Hkv, T_cap, 128), np.int8)
    mi.check(mi.lib.mi_kv_tiled_from_rows_i8(dkq.ptr, dvq.ptr, dkt.ptr, dvt.ptr, B * Hkv, T, T_cap, T_cap, None))
    dq = dev.upload(q)
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, 128, T_cap), np.uint8)
    dqq, dsq, ddots = dev.empty((B, Hq, 128), np.int8), dev.empty((B, Hq), np.float32), dev.empty((B, Hq, T), np.int32)
    mi.check(mi.lib.mi_gqa_decode_scores_tiled_i32(dq.ptr, dkt.ptr, dks.ptr, dvt.ptr, dvs.ptr, dqq.ptr, dsq.ptr, ddots.ptr,
                                                   B, Hq, Hkv, 128, T_cap, T, ws.ptr, ws.nbytes, None))
    assert np.array_equal(dev.download(dqq), gold["attn_qq"]) and np.array_equal(dev.download(dsq), gold["attn_sq"])
    assert np.array_equal(dev.download(ddots), gold["attn_dots"])
    do = dev.empty((B, Hq, 128), np.float32)
    dlen = dev.upload(np.full(B, T, np.int32))
    for rot, key in ((0, "attn_o"), (1, "attn_o_rot")):
        mi.check(mi.lib.mi_gqa_decode_attn_tiled(dq.ptr, dkt.ptr, dks.ptr, dvt.ptr, dvs.ptr, do.ptr, B, Hq, Hkv, 128, T_cap,
                                                 dlen.ptr, T, rot, ws.ptr, ws.nbytes, None))
        assert np.max(np.abs(dev.download(do) - gold[key])) <= 2e-5
    dev.reset_to(mark)


@pytest.mark.gpu
def test_gpu_moe(mi, dev, gold):
    mark = dev.mark()
    T, H, I, E, topk, _ = gen.MOE
    x, wr, wg, sg, wu, su, wd, sd = gen.moe_inputs()
    dx = dev.upload(x)
    didx, dw = dev.empty((T, topk), np.int32), dev.empty((T, topk), np.float32)
    rws = dev.empty(mi.lib.mi_moe_route_workspace_bytes(T, E), np.uint8)
    mi.moe_route(dx, dev.upload(wr), didx, dw, topk, rws)
    assert np.array_equal(dev.download(didx), gold["moe_idx"])
    assert np.max(np.abs(dev.download(dw) - gold["moe_w"])) <= 2e-6
    dperm, dseg = dev.empty(T * topk, np.int32), dev.empty(E + 1, np.int32)
    mi.moe_dispatch(dev.upload(gold["moe_idx"]), dperm, dseg, E)
    assert np.array_equal(dev.download(dperm), gold["moe_perm"]) and np.array_equal(dev.download(dseg), gold["moe_seg"])
    ws = dev.empty(mi.lib.mi_moe_ffn_workspace_bytes(T, H, I, E, topk), np.uint8)
    dy = dev.empty((T, H), np.float32)
    mi.moe_ffn(dx, dev.upload(gold["moe_idx"]), dev.upload(gold["moe_w"]), *(dev.upload(a) for a in (wg, sg, wu, su, wd, sd)),
               dy, ws)
    y = dev.download(dy)
    off = mi.lib.mi_moe_ffn_workspace_offset(4, T, H, I, E, topk)
    h = dev.download(ws.offset(off, (T * topk, I), np.float32))
    assert np.max(np.abs(h - gold["moe_h"])) <= 1e-5 * max(1.0, float(np.abs(gold["moe_h"]).max()))
    rel = np.linalg.norm(y.astype(np.float64) - gold["moe_y"]) / np.linalg.norm(gold["moe_y"].astype(np.float64))
    assert rel <= 1e-3
    dev.reset_to(mark)


@pytest.mark.gpu
def test_gpu_layer_ops(mi, dev, gold):
    mark = dev.mark()
    x, res, g, gu, eps = layer_inputs()
    R, W = x.shape
    dh, dy = dev.empty((R, W), np.float32), dev.empty((R, W), np.float32)
    mi.check(mi.lib.mi_rmsnorm_f32(dev.upload(x).ptr, dev.upload(res).ptr, dev.upload(g).ptr, eps, dh.ptr, dy.ptr, R, W, None))
    assert np.array_equal(dev.download(dh), gold["rms_h"])
    assert np.max(np.abs(dev.download(dy) - gold["rms_y"])) <= 2e-6 * float(np.abs(gold["rms_y"]).max())
    dsw = dev.empty((R, W), np.float32)
    mi.check(mi.lib.mi_swiglu_f32(dev.upload(gu).ptr, dsw.ptr, R, W, None))
    assert np.max(np.abs(dev.download(dsw) - gold["swiglu_h"])) <= 2e-6 * float(np.abs(gold["swiglu_h"]).max())
    # rotary embedding + cache append through the fused operator: one sequence per fixture row, one query head, one
    # key head and one value head that all carry the row; the sequence writes position pos[b] of its cache
    rows, npos, salt = gen.ROPE
    src = gen.bell((rows, 128), salt)
    pos = gold["rope_pos"]
    qkv = np.concatenate([src, src, src], axis=1)
    dq = dev.empty((rows, 1, 128), np.float32)
    zq, zs = np.zeros((rows, 1, npos, 128), np.int8), np.zeros((rows, 1, npos), np.float32)
    dkq, dks, dvq, dvs = dev.upload(zq), dev.upload(zs), dev.upload(zq), dev.upload(zs)
    mi.check(mi.lib.mi_rope_kv_append_f32_i8(dev.upload(qkv).ptr, qkv.shape[1], dev.upload(gold["rope_cos"]).ptr,
                                             dev.upload(gold["rope_sin"]).ptr, dq.ptr, dkq.ptr, dks.ptr, dvq.ptr, dvs.ptr,
                                             dev.upload(pos).ptr, rows, 1, 1, 128, npos, None))
    q, kq, ks, vq, vs = (dev.download(a) for a in (dq, dkq, dks, dvq, dvs))
    assert np.array_equal(q[:, 0], gold["rope_out"])
    for b in range(rows):
        assert np.array_equal(kq[b, 0, pos[b]], gold["rope_kq"][b]) and ks[b, 0, pos[b]] == gold["rope_ks"][b]
        assert np.array_equal(vq[b, 0, pos[b]], gold["rope_vq"][b]) and vs[b, 0, pos[b]] == gold["rope_vs"][b]
        others = np.delete(np.arange(npos), pos[b])
        assert not kq[b, 0, others].any() and not vq[b, 0, others].any()     # nothing else of the cache is touched
    dev.reset_to(mark)
