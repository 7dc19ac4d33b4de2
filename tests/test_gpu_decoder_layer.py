"""GPU parity: the fp32 operators between the int8 kernels of a decoder layer, and the whole layer of a decode
step against the oracle chain.  Gates: rotary embedding and the appended cache codes bit-exact; RMSNorm and SwiGLU
within 2e-6 relative (fp32 sums / expf against float64 / libm); layer output rel-L2 <= 1e-3."""
import numpy as np
import pytest

import workload
from test_oracle_layer_ops import rope_tables

pytestmark = pytest.mark.gpu
D = 128


@pytest.mark.parametrize("M,H", [(16, 4096), (1, 4096), (3, 14336), (5, 64), (2, 16384), (7, 1028)])
def test_rmsnorm_matches_oracle(mi, dev, orc, M, H):
    mark = dev.mark()
    g = np.random.default_rng(M * 7 + H)
    x = (g.standard_normal((M, H)) * 2).astype(np.float32)
    r = g.standard_normal((M, H)).astype(np.float32)
    w = (1 + 0.1 * g.standard_normal(H)).astype(np.float32)
    dx, dr, dw = dev.upload(x), dev.upload(r), dev.upload(w)
    dy, dh = dev.empty((M, H), np.float32), dev.empty((M, H), np.float32)
    mi.check(mi.lib.mi_rmsnorm_f32(dx.ptr, None, dw.ptr, 1e-5, None, dy.ptr, M, H, None))
    y = dev.download(dy)
    mi.check(mi.lib.mi_rmsnorm_f32(dx.ptr, dr.ptr, dw.ptr, 1e-5, dh.ptr, dy.ptr, M, H, None))
    h, y2 = dev.download(dh), dev.download(dy)
    dev.reset_to(mark)
    want = orc.rmsnorm(x, w, 1e-5)
    hw, want2 = orc.rmsnorm(x, w, 1e-5, residual=r)
    assert np.max(np.abs(y - want)) <= 2e-6 * np.max(np.abs(want))
    assert np.array_equal(h, hw)                                     # the residual sum is one fp32 add
    assert np.max(np.abs(y2 - want2)) <= 2e-6 * np.max(np.abs(want2))


def test_rmsnorm_refuses_bad_arguments(mi, dev):
    mark = dev.mark()
    x = dev.empty((2, 64), np.float32)
    lib = mi.lib
    assert lib.mi_rmsnorm_f32(x.ptr, None, x.ptr, 1e-5, None, x.ptr, 2, 62, None) == mi.EINVAL     # H % 4
    assert lib.mi_rmsnorm_f32(x.ptr, x.ptr, x.ptr, 1e-5, None, x.ptr, 2, 64, None) == mi.EINVAL    # residual without h_out
    assert lib.mi_rmsnorm_f32(x.ptr, None, x.ptr, 1e-5, None, x.ptr, 2, 32768, None) == mi.ERANGE
    assert lib.mi_rmsnorm_f32(x.ptr, None, x.ptr, -1.0, None, x.ptr, 2, 64, None) == mi.EINVAL
    dev.reset_to(mark)


@pytest.mark.parametrize("B,Hq,Hkv,T_cap,pad", [(16, 32, 8, 64, 0), (3, 4, 1, 20, 128), (1, 8, 8, 5, 0)])
def test_rope_kv_append_bit_exact(mi, dev, orc, B, Hq, Hkv, T_cap, pad):
    mark = dev.mark()
    g = np.random.default_rng(B + T_cap)
    heads = Hq + 2 * Hkv
    stride = heads * D + pad
    qkv = workload.normal(17, (B, stride), 0)
    cos, sin = rope_tables(T_cap)
    pos = g.integers(0, T_cap, B).astype(np.int32)
    if B > 2:
        pos[1] = T_cap                      # outside: nothing of this sequence is written
    bgq = g.integers(-127, 128, (B, Hkv, T_cap, D)).astype(np.int8)
    bgs = g.random((B, Hkv, T_cap), dtype=np.float32)
    q0 = workload.normal(18, (B, Hq, D), 0)
    dqkv, dcos, dsin, dpos = dev.upload(qkv), dev.upload(cos), dev.upload(sin), dev.upload(pos)
    dq = dev.upload(q0)
    dkq, dks, dvq, dvs = dev.upload(bgq), dev.upload(bgs), dev.upload(bgq), dev.upload(bgs)
    mi.check(mi.lib.mi_rope_kv_append_f32_i8(dqkv.ptr, stride, dcos.ptr, dsin.ptr, dq.ptr, dkq.ptr, dks.ptr, dvq.ptr,
                                             dvs.ptr, dpos.ptr, B, Hq, Hkv, D, T_cap, None))
    q, kq, ks, vq, vs = (dev.download(b) for b in (dq, dkq, dks, dvq, dvs))
    dev.reset_to(mark)
    wq, wkq, wks, wvq, wvs = q0.copy(), bgq.copy(), bgs.copy(), bgq.copy(), bgs.copy()
    for b in range(B):
        if not 0 <= pos[b] < T_cap:
            continue
        row = qkv[b, :heads * D].reshape(heads, D)
        pp = np.full(Hq + Hkv, pos[b], np.int32)
        roped = orc.rope_rows(row[:Hq + Hkv], pp, cos, sin)
        wq[b] = roped[:Hq]
        kc, ksc = orc.rotate_quant_rows(roped[Hq:], D)
        vc, vsc = orc.rotate_quant_rows(np.ascontiguousarray(row[Hq + Hkv:]), D)
        wkq[b, :, pos[b]], wks[b, :, pos[b]] = kc, ksc
        wvq[b, :, pos[b]], wvs[b, :, pos[b]] = vc, vsc
    assert np.array_equal(q, wq)
    assert np.array_equal(kq, wkq) and np.array_equal(ks, wks)
    assert np.array_equal(vq, wvq) and np.array_equal(vs, wvs)


@pytest.mark.parametrize("M,I", [(16, 14336), (1, 768), (5, 4)])
def test_swiglu_matches_oracle(mi, dev, orc, M, I):
    mark = dev.mark()
    gu = (workload.normal(23, (M, 2 * I), 0) * 3).astype(np.float32)
    dgu, dh = dev.upload(gu), dev.empty((M, I), np.float32)
    mi.check(mi.lib.mi_swiglu_f32(dgu.ptr, dh.ptr, M, I, None))
    h = dev.download(dh)
    dev.reset_to(mark)
    want = orc.swiglu(gu)
    assert np.max(np.abs(h - want)) <= 2e-6 * max(1.0, np.max(np.abs(want)))


def test_add(mi, dev):
    mark = dev.mark()
    a, b = workload.normal(1, (3, 1024), 0), workload.normal(1, (3, 1024), 1)
    da, db, dc = dev.upload(a), dev.upload(b), dev.empty((3, 1024), np.float32)
    mi.check(mi.lib.mi_add_f32(da.ptr, db.ptr, dc.ptr, a.size, None))
    c = dev.download(dc)
    dev.reset_to(mark)
    assert np.array_equal(c, a + b)


def rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b) / max(float(np.linalg.norm(b)), 1e-30))


def oracle_layer(orc, x, W, cache, pos, lens, cos, sin, eps, Hq, Hkv, gpu=None, moe=None):
    """The same chain on the CPU oracle; `cache` = [kq, ks, vq, vs] numpy arrays, updated in place.

    With `gpu` (the GPU's own intermediates by name) every stage is fed what the GPU fed its next kernel and is
    checked on its own: a rounding tie met from the other side of an ulp flips an int8 code, and a chain of
    quantizers turns a dense 1e-7 difference into sparse one-code differences that grow from linear to linear,
    so only stage-wise parity can be tight (integer stages bit-exact, fp32 stages to their stated tolerance)."""
    B, H = x.shape
    heads = Hq + 2 * Hkv
    take = (lambda name, own: gpu[name]) if gpu is not None else (lambda name, own: own)
    xn = orc.rmsnorm(x, W["g1"], eps)
    if gpu is not None:
        assert np.max(np.abs(gpu["xn"] - xn)) <= 2e-6 * np.max(np.abs(xn))
    qkv = orc.w8a8_linear(take("xn", xn), W["qkv"][0], W["qkv"][1], 128)[0]
    if gpu is not None:
        assert np.array_equal(gpu["qkv"], qkv)
    qkv = take("qkv", qkv)
    q = np.empty((B, Hq, D), np.float32)
    for b in range(B):
        row = qkv[b].reshape(heads, D)
        roped = orc.rope_rows(row[:Hq + Hkv], np.full(Hq + Hkv, pos[b], np.int32), cos, sin)
        q[b] = roped[:Hq]
        cache[0][b, :, pos[b]], cache[1][b, :, pos[b]] = orc.rotate_quant_rows(roped[Hq:], D)
        cache[2][b, :, pos[b]], cache[3][b, :, pos[b]] = orc.rotate_quant_rows(np.ascontiguousarray(row[Hq + Hkv:]), D)
    if gpu is not None:
        assert np.array_equal(gpu["q"], q)
        for name, ref in zip(("kq", "ks", "vq", "vs"), cache):
            assert np.array_equal(gpu[name], ref)
    att = np.empty((B, Hq, D), np.float32)
    for b in range(B):
        n = int(lens[b])
        att[b] = orc.gqa_decode(q[b:b + 1], *(np.ascontiguousarray(c[b:b + 1, :, :n]) for c in cache),
                                out_rotated=True)[0]
    att = att.reshape(B, Hq * D)
    if gpu is not None:
        assert np.max(np.abs(gpu["att"] - att)) <= 2e-5          # gate 2e-3
    # the O projection takes the attention row as it stands in the rotated basis: quantized per token, no rotation
    a = take("att", att)
    qa = np.empty((B, Hq * D), np.int8)
    sa = np.empty(B, np.float32)
    for b in range(B):
        qa[b], sa[b] = orc.quant_row(a[b])
    if gpu is not None:
        assert np.array_equal(gpu["ca"], qa) and np.array_equal(gpu["sa"], sa)
    ao = orc.dequant(orc.gemm_i8_i32(qa, W["o"][0]), sa, W["o"][1])
    if gpu is not None:
        assert np.array_equal(gpu["ao"], ao)
    h1, hn = orc.rmsnorm(take("ao", ao), W["g2"], eps, residual=x)
    if gpu is not None:
        assert np.array_equal(gpu["h1"], h1)
        assert np.max(np.abs(gpu["hn"] - hn)) <= 2e-6 * np.max(np.abs(hn))
    if moe is not None:
        # the FFN half is router + dispatch + grouped experts on the normalized row (a9-a11)
        xin = take("hn", hn)
        idx, w = orc.moe_route(xin, moe["wr"], moe["topk"])
        if gpu is not None:
            assert np.array_equal(gpu["moe_idx"], idx)
            assert np.max(np.abs(gpu["moe_w"] - w)) <= 2e-6
            idx, w = gpu["moe_idx"], gpu["moe_w"]
        dn = orc.moe_ffn(xin, idx, w, moe["wg"], moe["sg"], moe["wu"], moe["su"], moe["wd"], moe["sd"], 128, 256)
        if gpu is not None:
            assert rel(gpu["dn"], dn) <= 1e-3          # SwiGLU goes through expf: the stated gate of the FFN output
        return take("h1", h1) + take("dn", dn)
    gu = orc.w8a8_linear(take("hn", hn), W["gu"][0], W["gu"][1], 128)[0]
    if gpu is not None:
        assert np.array_equal(gpu["gu"], gu)
    act = orc.swiglu(take("gu", gu))
    if gpu is not None:
        assert np.max(np.abs(gpu["act"] - act)) <= 2e-6 * max(1.0, float(np.max(np.abs(act))))
    dn = orc.w8a8_linear(take("act", act), W["d"][0], W["d"][1], 128)[0]
    if gpu is not None:
        assert np.array_equal(gpu["dn"], dn)
    return take("h1", h1) + take("dn", dn)


@pytest.mark.parametrize("B,H,Hq,Hkv,I,T_cap,start", [
    (4, 1024, 8, 2, 2048, 64, [0, 10, 40, 61]),
    (2, 4096, 32, 8, 14336, 300, [150, 297]),
    (16, 4096, 32, 8, 14336, 128, list(range(100, 116))),
    (1, 4096, 32, 8, 14336, 600, [500]),          # one sequence: the norm-fused GEMVs and the short attention spans
    (1, 2048, 8, 2, 1024, 40, [7]),
])
def test_decoder_layer_decode_steps_follow_the_oracle_chain(mi, dev, orc, B, H, Hq, Hkv, I, T_cap, start):
    mark = dev.mark()
    eps = 1e-5
    cos, sin = rope_tables(T_cap)
    fw = {"qkv": workload.weights(41, (Hq + 2 * Hkv) * D, H, 1), "o": workload.weights(41, H, Hq * D, 2),
          "gu": workload.weights(41, 2 * I, H, 3), "d": workload.weights(41, H, I, 4)}
    g = np.random.default_rng(41)
    g1 = (1 + 0.1 * g.standard_normal(H)).astype(np.float32)
    g2 = (1 + 0.1 * g.standard_normal(H)).astype(np.float32)
    layer = mi.DecoderLayer(dev, B, H, Hq, Hkv, I, T_cap, fw["qkv"], fw["o"], fw["gu"], fw["d"], g1, g2, cos, sin, eps,
                            trace=True, tiled=T_cap % 64 == 0)
    W = {k: orc.rotate_quant_rows(v, 128) for k, v in fw.items()}
    for k, dv in (("qkv", layer.wqkv), ("o", layer.wo), ("gu", layer.wgu), ("d", layer.wd)):
        assert np.array_equal(dev.download(dv[0]), W[k][0]) and np.array_equal(dev.download(dv[1]), W[k][1])
    W["g1"], W["g2"] = g1, g2
    # prefixes: random codes with sane scales, the same on both sides
    start = np.array(start, np.int32)
    cache = [g.integers(-127, 128, (B, Hkv, T_cap, D)).astype(np.int8),
             ((g.random((B, Hkv, T_cap)) + 0.5) * 0.03).astype(np.float32),
             g.integers(-127, 128, (B, Hkv, T_cap, D)).astype(np.int8),
             ((g.random((B, Hkv, T_cap)) + 0.5) * 0.03).astype(np.float32)]
    free = [c.copy() for c in cache]
    assert layer.tiled == (T_cap % 64 == 0)      # capacities of 64 and 128 tokens run the matrix-pipe layouts
    layer.set_cache_rows(*cache)
    dpos, dlen = dev.empty(B, np.int32), dev.empty(B, np.int32)
    dx, dout = dev.empty((B, H), np.float32), dev.empty((B, H), np.float32)
    names = ("xn", "qkv", "q", "att", "ca", "sa", "ao", "h1", "hn", "gu", "act", "dn")

    def snapshot():
        got = {n: dev.download(getattr(layer, n)) for n in names}
        got["kq"], got["ks"], got["vq"], got["vs"] = layer.get_cache_rows()
        return got
    for step in range(3):
        pos = (start + step).astype(np.int32)
        lens = (pos + 1).astype(np.int32)
        x = workload.activations(300 + step, B, H)
        for d, a in ((dpos, pos), (dlen, lens), (dx, x)):
            mi.check(mi.lib.mi_memcpy_h2d(d.ptr, a.ctypes.data, a.nbytes, None))
        layer.step(dx, dpos, dlen, int(lens.max()), dout)
        out = dev.download(dout)
        gpu = snapshot()
        gpu["q"] = gpu["q"].reshape(B, Hq, D)
        # stage by stage, each stage fed what the GPU fed it: integer stages bit-exact
        staged = oracle_layer(orc, x, W, cache, pos, lens, cos, sin, eps, Hq, Hkv, gpu=gpu)
        assert np.array_equal(out, staged)
        # the free-running oracle chain: same result up to the code flips that ulp-level differences cause in
        # five quantizers in a row (measured 2e-4 .. 6e-3)
        want = oracle_layer(orc, x, W, free, pos, lens, cos, sin, eps, Hq, Hkv)
        assert rel(out, want) <= 3e-2, "step %d rel-L2 %.3e" % (step, rel(out, want))
    # the layer fed as the next layer of a stack is fed: input = down output + residual of the layer before, the
    # closing add left to the layer after (out=None); positions that do not collide with the steps above
    prev_dn, prev_h1 = dev.download(layer.dn), dev.download(layer.h1)
    d_dn, d_h1 = dev.upload(prev_dn), dev.upload(prev_h1)
    pos = np.minimum(start + 3, T_cap - 1).astype(np.int32)
    lens = (pos + 1).astype(np.int32)
    for d, a in ((dpos, pos), (dlen, lens)):
        mi.check(mi.lib.mi_memcpy_h2d(d.ptr, a.ctypes.data, a.nbytes, None))
    layer.step(d_dn, dpos, dlen, int(lens.max()), None, residual=d_h1)
    gpu = snapshot()
    gpu["q"] = gpu["q"].reshape(B, Hq, D)
    x_in = prev_dn + prev_h1
    assert np.array_equal(dev.download(layer.h0), x_in)
    staged = oracle_layer(orc, x_in, W, cache, pos, lens, cos, sin, eps, Hq, Hkv, gpu=gpu)
    assert np.array_equal(gpu["h1"] + gpu["dn"], staged)
    dev.reset_to(mark)


@pytest.mark.parametrize("M,H,block", [(16, 4096, 128), (3, 14336, 128), (2, 768, 256), (1, 128, 128), (5, 16384, 256)])
def test_fused_rmsnorm_quant_equals_the_two_calls(mi, dev, orc, M, H, block):
    """Codes and scales of the fused kernel = the stand-alone quantizer applied to the fp32 row the fused kernel
    reports, and that row follows the RMSNorm oracle; the residual sum is one fp32 add."""
    mark = dev.mark()
    g = np.random.default_rng(M + H)
    x = workload.activations(61, M, H)
    r = g.standard_normal((M, H)).astype(np.float32)
    w = (1 + 0.1 * g.standard_normal(H)).astype(np.float32)
    dx, dr, dw = dev.upload(x), dev.upload(r), dev.upload(w)
    dh, dy = dev.empty((M, H), np.float32), dev.empty((M, H), np.float32)
    dq, ds = dev.empty((M, H), np.int8), dev.empty(M, np.float32)
    for res in (None, dr):
        mi.check(mi.lib.mi_rmsnorm_quant_f32_i8(dx.ptr, res.ptr if res else None, dw.ptr, 1e-5,
                                                dh.ptr if res else None, dy.ptr, dq.ptr, ds.ptr, M, H, block, None))
        y, q, sc = dev.download(dy), dev.download(dq), dev.download(ds)
        xin = x + r if res else x
        if res:
            assert np.array_equal(dev.download(dh), xin)
        want = orc.rmsnorm(xin, w, 1e-5)
        assert np.max(np.abs(y - want)) <= 2e-6 * np.max(np.abs(want))
        qo, so = orc.rotate_quant_rows(y, block)
        assert np.array_equal(q, qo) and np.array_equal(sc, so)
        # without the fp32 row: same codes
        mi.check(mi.lib.mi_rmsnorm_quant_f32_i8(dx.ptr, res.ptr if res else None, dw.ptr, 1e-5,
                                                dh.ptr if res else None, None, dq.ptr, ds.ptr, M, H, block, None))
        assert np.array_equal(dev.download(dq), qo) and np.array_equal(dev.download(ds), so)
    dev.reset_to(mark)


@pytest.mark.parametrize("M,I,block", [(16, 14336, 128), (4, 768, 256), (1, 256, 128)])
def test_fused_swiglu_quant_equals_the_two_calls(mi, dev, orc, M, I, block):
    mark = dev.mark()
    gu = (workload.normal(29, (M, 2 * I), 0) * 2).astype(np.float32)
    dgu, dh = dev.upload(gu), dev.empty((M, I), np.float32)
    dq, ds = dev.empty((M, I), np.int8), dev.empty(M, np.float32)
    mi.check(mi.lib.mi_swiglu_quant_f32_i8(dgu.ptr, dh.ptr, dq.ptr, ds.ptr, M, I, block, None))
    h, q, sc = dev.download(dh), dev.download(dq), dev.download(ds)
    want = orc.swiglu(gu)
    assert np.max(np.abs(h - want)) <= 2e-6 * max(1.0, float(np.max(np.abs(want))))
    qo, so = orc.rotate_quant_rows(h, block)
    assert np.array_equal(q, qo) and np.array_equal(sc, so)
    mi.check(mi.lib.mi_swiglu_quant_f32_i8(dgu.ptr, None, dq.ptr, ds.ptr, M, I, block, None))
    assert np.array_equal(dev.download(dq), qo) and np.array_equal(dev.download(ds), so)
    assert mi.lib.mi_swiglu_quant_f32_i8(dgu.ptr, None, dq.ptr, ds.ptr, M, I + 4, block, None) == mi.EINVAL
    dev.reset_to(mark)


@pytest.mark.parametrize("M,N,K", [(1, 6144, 4096), (1, 28672, 4096), (1, 272, 2048), (1, 512, 1024), (3, 1024, 4096),
                                   (16, 512, 14336)])
def test_rmsnorm_linear_one_call(mi, dev, orc, M, N, K):
    """One token and K in {2048, 4096}: a single kernel; other shapes: norm + quantize, then the contraction.  Either
    way the normalized row follows the RMSNorm oracle, the codes are the oracle quantizer's on that row and the
    output is the oracle's contraction of those codes, exactly."""
    mark = dev.mark()
    g = np.random.default_rng(M + N + K)
    x = workload.activations(71, M, K)
    r = g.standard_normal((M, K)).astype(np.float32)
    w = (1 + 0.1 * g.standard_normal(K)).astype(np.float32)
    qw = g.integers(-127, 128, (N, K)).astype(np.int8)
    sw = ((g.random(N) + 0.5) * 0.01).astype(np.float32)
    dx, dr, dg, dqw, dsw = dev.upload(x), dev.upload(r), dev.upload(w), dev.upload(qw), dev.upload(sw)
    dh, dxn, dy = dev.empty((M, K), np.float32), dev.empty((M, K), np.float32), dev.empty((M, N), np.float32)
    ws = dev.empty(mi.lib.mi_w8a8_linear_workspace_bytes(M, N, K), np.uint8)
    for res in (None, dr):
        for want_xn in (True, False):
            mi.check(mi.lib.mi_rmsnorm_linear_f32(dx.ptr, res.ptr if res else None, dg.ptr, 1e-5, dh.ptr if res else None,
                                                  dxn.ptr if want_xn else None, dqw.ptr, dsw.ptr, dy.ptr, M, N, K, 128,
                                                  ws.ptr, ws.nbytes, None), "mi_rmsnorm_linear_f32")
            y = dev.download(dy)
            xin = x + r if res else x
            if res:
                assert np.array_equal(dev.download(dh), xin)
            if want_xn:
                xn = dev.download(dxn)
                ref = orc.rmsnorm(xin, w, 1e-5)
                assert np.max(np.abs(xn - ref)) <= 2e-6 * np.max(np.abs(ref))
                want = orc.w8a8_linear(xn, qw, sw, 128)
                assert np.array_equal(dev.download(ws.offset(0, (M, K), np.int8)), want[1])
                y_first = y
                assert np.array_equal(y, want[0])
            else:
                assert np.array_equal(y, y_first)          # leaving the fp32 row out changes nothing
    assert mi.lib.mi_rmsnorm_linear_f32(dx.ptr, dr.ptr, dg.ptr, 1e-5, None, None, dqw.ptr, dsw.ptr, dy.ptr, M, N, K, 128,
                                        ws.ptr, ws.nbytes, None) == mi.EINVAL     # residual without h_out
    dev.reset_to(mark)


@pytest.mark.parametrize("M,N,K", [(1, 6144, 4096), (1, 272, 2048), (4, 512, 4096)])
@pytest.mark.parametrize("target", ["residual", "x"])
def test_rmsnorm_linear_residual_stream_updated_in_place(mi, dev, orc, M, N, K, target):
    """h_out written over the residual (or over x), the way a decoder updates its residual stream: the one-kernel
    form reads both rows in every workgroup, so such a call has to give what separate buffers give."""
    mark = dev.mark()
    g = np.random.default_rng(5 * M + N + K)
    x = workload.activations(72, M, K)
    r = g.standard_normal((M, K)).astype(np.float32)
    w = (1 + 0.1 * g.standard_normal(K)).astype(np.float32)
    qw = g.integers(-127, 128, (N, K)).astype(np.int8)
    sw = ((g.random(N) + 0.5) * 0.01).astype(np.float32)
    dx, dr, dg, dqw, dsw = dev.upload(x), dev.upload(r), dev.upload(w), dev.upload(qw), dev.upload(sw)
    dh, dy, dy2 = dev.empty((M, K), np.float32), dev.empty((M, N), np.float32), dev.empty((M, N), np.float32)
    ws = dev.empty(mi.lib.mi_w8a8_linear_workspace_bytes(M, N, K), np.uint8)
    mi.check(mi.lib.mi_rmsnorm_linear_f32(dx.ptr, dr.ptr, dg.ptr, 1e-5, dh.ptr, None, dqw.ptr, dsw.ptr, dy.ptr, M, N, K,
                                          128, ws.ptr, ws.nbytes, None), "separate buffers")
    y_sep, h_sep = dev.download(dy), dev.download(dh)
    codes_sep = dev.download(ws.offset(0, (M, K), np.int8))
    for _ in range(3):   # the race needs workgroups to start after the keeper has written: several tries, each from fresh rows
        mi.check(mi.lib.mi_memcpy_h2d(dx.ptr, x.ctypes.data, x.nbytes, None))
        mi.check(mi.lib.mi_memcpy_h2d(dr.ptr, r.ctypes.data, r.nbytes, None))
        dev.sync()
        dst = dr if target == "residual" else dx
        mi.check(mi.lib.mi_rmsnorm_linear_f32(dx.ptr, dr.ptr, dg.ptr, 1e-5, dst.ptr, None, dqw.ptr, dsw.ptr, dy2.ptr, M, N,
                                              K, 128, ws.ptr, ws.nbytes, None), "in place")
        assert np.array_equal(dev.download(dst), h_sep)
        assert np.array_equal(dev.download(ws.offset(0, (M, K), np.int8)), codes_sep)
        assert np.array_equal(dev.download(dy2), y_sep)
    dev.reset_to(mark)


@pytest.mark.parametrize("K", [2048, 4096])
def test_one_token_gets_the_same_codes_alone_and_in_a_batch(mi, dev, K):
    """The one-kernel form (M = 1) and the row operator (M > 1) sum the squares in the same order: a token's
    normalized row, codes and scale do not depend on the batch it arrives in."""
    mark = dev.mark()
    N = 256
    g = np.random.default_rng(K)
    x = workload.activations(73, 3, K)
    r = g.standard_normal((3, K)).astype(np.float32)
    w = (1 + 0.1 * g.standard_normal(K)).astype(np.float32)
    qw = g.integers(-127, 128, (N, K)).astype(np.int8)
    sw = ((g.random(N) + 0.5) * 0.01).astype(np.float32)
    dg, dqw, dsw = dev.upload(w), dev.upload(qw), dev.upload(sw)
    ws = dev.empty(mi.lib.mi_w8a8_linear_workspace_bytes(3, N, K), np.uint8)

    def run(rows):
        M = len(rows)
        dx, dr = dev.upload(x[rows]), dev.upload(r[rows])
        dh, dxn, dy = dev.empty((M, K), np.float32), dev.empty((M, K), np.float32), dev.empty((M, N), np.float32)
        mi.check(mi.lib.mi_rmsnorm_linear_f32(dx.ptr, dr.ptr, dg.ptr, 1e-5, dh.ptr, dxn.ptr, dqw.ptr, dsw.ptr, dy.ptr, M, N,
                                              K, 128, ws.ptr, ws.nbytes, None), "mi_rmsnorm_linear_f32")
        sx_off = (M * K + 255) // 256 * 256
        return (dev.download(dxn), dev.download(ws.offset(0, (M, K), np.int8)),
                dev.download(ws.offset(sx_off, (M,), np.float32)), dev.download(dy))
    batch = run([0, 1, 2])
    for m in range(3):
        alone = run([m])
        for a, b in zip(alone, batch):
            assert np.array_equal(a[0], b[m])
    dev.reset_to(mark)


@pytest.mark.parametrize("B,H,Hq,Hkv,I,E,topk,T_cap,start", [
    (3, 512, 4, 2, 256, 16, 2, 40, [0, 17, 38]),
    (16, 2048, 16, 4, 768, 128, 8, 128, list(range(90, 106))),      # the cfg4 experts behind a 16-sequence decode step
])
def test_moe_decoder_layer_decode_steps_follow_the_oracle_chain(mi, dev, orc, B, H, Hq, Hkv, I, E, topk, T_cap, start):
    """The decoder layer with the MoE FFN in place of the dense one: attention half as above, then residual + RMSNorm,
    router (indices exact, weights to 2e-6), dispatch and grouped expert FFN (rel-L2 1e-3 against the oracle fed the
    GPU's routing), residual."""
    mark = dev.mark()
    eps = 1e-5
    cos, sin = rope_tables(T_cap)
    fw = {"qkv": workload.weights(43, (Hq + 2 * Hkv) * D, H, 1), "o": workload.weights(43, H, Hq * D, 2)}
    g = np.random.default_rng(43)
    g1 = (1 + 0.1 * g.standard_normal(H)).astype(np.float32)
    g2 = (1 + 0.1 * g.standard_normal(H)).astype(np.float32)
    moe = {"wr": workload.weights(44, E, H), "topk": topk}
    for name, n, k, b in (("g", I, H, 128), ("u", I, H, 128), ("d", H, I, 256)):
        q, sc = orc.rotate_quant_rows(workload.weights(45, E * n, k, len(name) + n), b)
        moe["w" + name], moe["s" + name] = q.reshape(E, n, k), sc.reshape(E, n)
    layer = mi.DecoderLayer(dev, B, H, Hq, Hkv, I, T_cap, fw["qkv"], fw["o"], None, None, g1, g2, cos, sin, eps,
                            trace=True, tiled=T_cap % 64 == 0, moe=moe)
    W = {k: orc.rotate_quant_rows(v, 128) for k, v in fw.items()}
    W["g1"], W["g2"] = g1, g2
    start = np.array(start, np.int32)
    cache = [g.integers(-127, 128, (B, Hkv, T_cap, D)).astype(np.int8),
             ((g.random((B, Hkv, T_cap)) + 0.5) * 0.03).astype(np.float32),
             g.integers(-127, 128, (B, Hkv, T_cap, D)).astype(np.int8),
             ((g.random((B, Hkv, T_cap)) + 0.5) * 0.03).astype(np.float32)]
    layer.set_cache_rows(*cache)
    dpos, dlen = dev.empty(B, np.int32), dev.empty(B, np.int32)
    dx, dout = dev.empty((B, H), np.float32), dev.empty((B, H), np.float32)
    names = ("xn", "qkv", "q", "att", "ca", "sa", "ao", "h1", "hn", "dn")
    off = lambda i: mi.lib.mi_moe_ffn_workspace_offset(i, B, H, I, E, topk)
    for step in range(2):
        pos = (start + step).astype(np.int32)
        lens = (pos + 1).astype(np.int32)
        x = workload.activations(310 + step, B, H)
        for d, a in ((dpos, pos), (dlen, lens), (dx, x)):
            mi.check(mi.lib.mi_memcpy_h2d(d.ptr, a.ctypes.data, a.nbytes, None))
        layer.step(dx, dpos, dlen, int(lens.max()), dout)
        out = dev.download(dout)
        gpu = {n: dev.download(getattr(layer, n)) for n in names}
        gpu["kq"], gpu["ks"], gpu["vq"], gpu["vs"] = layer.get_cache_rows()
        gpu["q"] = gpu["q"].reshape(B, Hq, D)
        gpu["moe_idx"] = dev.download(layer.moe_ws.offset(off(8), (B, topk), np.int32))
        gpu["moe_w"] = dev.download(layer.moe_ws.offset(off(9), (B, topk), np.float32))
        staged = oracle_layer(orc, x, W, cache, pos, lens, cos, sin, eps, Hq, Hkv, gpu=gpu, moe=moe)
        assert np.array_equal(out, staged)
        assert np.all(np.isfinite(out))
    dev.reset_to(mark)
