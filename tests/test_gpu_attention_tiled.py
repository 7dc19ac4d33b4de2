"""GPU parity: GQA decode attention over the cache in the matrix-pipe layouts (keys in 16-token tiles, values in
transposed 64-token blocks; both products on the int8 matrix pipe), the layout converter and the append kernels.
Gates: output max-abs <= 2e-3 against the oracle (in fact <= 2e-5); converter and appended codes bit-exact."""
import numpy as np
import pytest

import workload

pytestmark = pytest.mark.gpu

TOL = 2e-3


def to_blocks(vq, T_cap):
    """numpy restatement of the value layout: [B,Hkv,T,128] -> [B,Hkv,T_cap/64, 8,4,16,16] (kept as [.., 128, 64])"""
    B, Hkv, T, D = vq.shape
    pad = np.zeros((B, Hkv, T_cap, D), np.int8)
    pad[:, :, :T] = vq
    # token = 64*blk + 16*tc + tb, dim = 16*dp + dr  ->  (blk, dp, tc, dr, tb)
    x = pad.reshape(B, Hkv, T_cap // 64, 4, 16, 8, 16).transpose(0, 1, 2, 5, 3, 6, 4)
    return np.ascontiguousarray(x).reshape(B, Hkv, T_cap // 64, 128, 64)


def to_tiles(kq, T_cap):
    """numpy restatement of the key layout: [B,Hkv,T,128] -> [B,Hkv,T_cap/16,8,16,16] (chunk, token, byte)"""
    B, Hkv, T, D = kq.shape
    pad = np.zeros((B, Hkv, T_cap, D), np.int8)
    pad[:, :, :T] = kq
    return np.ascontiguousarray(pad.reshape(B, Hkv, T_cap // 16, 16, 8, 16).transpose(0, 1, 2, 4, 3, 5))


def from_tiles(kt):
    B, Hkv, nt = kt.shape[:3]
    return np.ascontiguousarray(kt.transpose(0, 1, 2, 4, 3, 5)).reshape(B, Hkv, nt * 16, 128)


def from_blocks(vt):
    B, Hkv, nb = vt.shape[:3]
    x = vt.reshape(B, Hkv, nb, 8, 4, 16, 16).transpose(0, 1, 2, 4, 6, 3, 5)   # (blk, tc, tb, dp, dr)
    return np.ascontiguousarray(x).reshape(B, Hkv, nb * 64, 128)


def convert(mi, dev, kq, vq, T, T_cap, junk_seed=None):
    """device converter on row-major codes [B,Hkv,T,128]; returns (dkt, dvt)"""
    B, Hkv = kq.shape[:2]
    dkq, dvq = dev.upload(kq), dev.upload(vq)
    if junk_seed is None:
        dkt, dvt = dev.empty((B, Hkv, T_cap // 16, 8, 16, 16), np.int8), dev.empty((B, Hkv, T_cap // 64, 128, 64), np.int8)
    else:
        g = np.random.default_rng(junk_seed)
        dkt = dev.upload(g.integers(-127, 128, (B, Hkv, T_cap // 16, 8, 16, 16)).astype(np.int8))
        dvt = dev.upload(g.integers(-127, 128, (B, Hkv, T_cap // 64, 128, 64)).astype(np.int8))
    mi.check(mi.lib.mi_kv_tiled_from_rows_i8(dkq.ptr, dvq.ptr, dkt.ptr, dvt.ptr, B * Hkv, T, kq.shape[2], T_cap, None),
             "mi_kv_tiled_from_rows_i8")
    return dkt, dvt


def make_cache(mi, dev, seed, B, Hq, Hkv, T, T_cap):
    D = 128
    q = workload.normal(seed, (B, Hq, D), 0)
    k = workload.normal(seed, (B * Hkv * T, D), 1)
    v = workload.normal(seed, (B * Hkv * T, D), 2)
    dk, dv = dev.upload(k), dev.upload(v)
    dkq, dks = dev.empty((B, Hkv, T, D), np.int8), dev.empty((B, Hkv, T), np.float32)
    dvq, dvs = dev.empty((B, Hkv, T, D), np.int8), dev.empty((B, Hkv, T), np.float32)
    mi.check(mi.lib.mi_fwht_quant_f32_i8(dk.ptr, dkq.ptr, dks.ptr, B * Hkv * T, D, D, None))
    mi.check(mi.lib.mi_fwht_quant_f32_i8(dv.ptr, dvq.ptr, dvs.ptr, B * Hkv * T, D, D, None))
    kq, ks, vq, vs = (dev.download(b) for b in (dkq, dks, dvq, dvs))
    # the cache proper: capacity T_cap per row, the tail filled with junk that must never be used
    ks_c = np.full((B, Hkv, T_cap), np.nan, np.float32)
    vs_c = np.full((B, Hkv, T_cap), np.nan, np.float32)
    ks_c[:, :, :T], vs_c[:, :, :T] = ks, vs
    return q, kq, ks, vq, vs, ks_c, vs_c


@pytest.mark.parametrize("B,Hq,Hkv,T,T_cap", [
    (2, 8, 2, 256, 256), (1, 4, 1, 16, 64), (1, 32, 8, 1000, 1024), (3, 6, 3, 77, 128), (2, 4, 4, 130, 192),
    (1, 8, 2, 1, 64), (1, 8, 2, 4096, 4096), (16, 32, 8, 700, 1024), (2, 8, 8, 64, 64),
    (1, 32, 8, 2000, 2048), (2, 16, 4, 1500, 1536),     # 32 and 24 splits: the merge with 32 lanes per row
])
def test_vt_attention_matches_oracle(mi, dev, orc, B, Hq, Hkv, T, T_cap):
    mark = dev.mark()
    q, kq, ks, vq, vs, ks_c, vs_c = make_cache(mi, dev, 300 + T, B, Hq, Hkv, T, T_cap)
    # the converter against the numpy restatement of the layouts (junk in the destination beforehand, which stays
    # in the blocks past the last one touched and must never be used)
    dkq, dvt = convert(mi, dev, kq, vq, T, T_cap, junk_seed=1)
    nb = (T + 63) // 64
    assert np.array_equal(dev.download(dvt)[:, :, :nb], to_blocks(vq, T_cap)[:, :, :nb])
    assert np.array_equal(dev.download(dkq)[:, :, :4 * nb], to_tiles(kq, T_cap)[:, :, :4 * nb])
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, 128, T_cap), np.uint8)
    dq, dks, dvs = dev.upload(q), dev.upload(ks_c), dev.upload(vs_c)
    do = dev.empty((B, Hq, 128), np.float32)
    for out_rotated in (False, True):
        oo = orc.gqa_decode(q, kq, ks, vq, vs, out_rotated=out_rotated)
        for lens in (None, np.full(B, T, np.int32)):
            mi.check(mi.lib.mi_fill_u32(do.ptr, 0x7fc00000, B * Hq * 128, None))
            dl = dev.upload(lens) if lens is not None else None
            # without lengths every sequence holds T_max = T tokens
            mi.check(mi.lib.mi_gqa_decode_attn_tiled(dq.ptr, dkq.ptr, dks.ptr, dvt.ptr, dvs.ptr, do.ptr, B, Hq, Hkv, 128,
                                                  T_cap, dl.ptr if dl else None, T, 1 if out_rotated else 0, ws.ptr,
                                                  ws.nbytes, None), "mi_gqa_decode_attn_tiled")
            o = dev.download(do)
            assert np.max(np.abs(o - oo)) <= TOL
            assert np.max(np.abs(o - oo)) <= 2e-5     # fixed-point weights of 28 bits: as good as fp32 accumulation
    dev.reset_to(mark)


def test_vt_ragged_lengths_and_zero_length(mi, dev, orc):
    """Per-sequence lengths inside one call, one of them 0 (a row of zeros), one of them 1, one full."""
    mark = dev.mark()
    B, Hq, Hkv, T_cap = 5, 8, 2, 512
    lens = np.array([512, 0, 1, 65, 300], np.int32)
    q, kq, ks, vq, vs, _, _ = make_cache(mi, dev, 17, B, Hq, Hkv, T_cap, T_cap)
    dkq, dvt = convert(mi, dev, kq, vq, T_cap, T_cap)
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, 128, T_cap), np.uint8)
    dq, dks, dvs, dl = dev.upload(q), dev.upload(ks), dev.upload(vs), dev.upload(lens)
    do = dev.empty((B, Hq, 128), np.float32)
    mi.check(mi.lib.mi_gqa_decode_attn_tiled(dq.ptr, dkq.ptr, dks.ptr, dvt.ptr, dvs.ptr, do.ptr, B, Hq, Hkv, 128, T_cap,
                                          dl.ptr, T_cap, 0, ws.ptr, ws.nbytes, None))
    o = dev.download(do)
    dev.reset_to(mark)
    for b in range(B):
        n = int(lens[b])
        if n == 0:
            assert np.all(o[b] == 0)
            continue
        oo = orc.gqa_decode(q[b:b + 1], kq[b:b + 1, :, :n], ks[b:b + 1, :, :n], vq[b:b + 1, :, :n], vs[b:b + 1, :, :n])
        assert np.max(np.abs(o[b] - oo[0])) <= 2e-5, b


def test_vt_peaked_and_flat_softmax(mi, dev, orc):
    """The fixed-point weights at their extremes: one token takes all the weight (its key is the query scaled up),
    and all tokens weigh the same (identical keys); V scales spread over three decades inside one span."""
    mark = dev.mark()
    B, Hq, Hkv, T, D = 1, 4, 1, 1024, 128
    g = np.random.default_rng(5)
    q = g.standard_normal((B, Hq, D)).astype(np.float32)
    v = (g.standard_normal((T, D)) * np.exp(g.uniform(-3.5, 3.5, (T, 1)))).astype(np.float32)
    for mode in ("peaked", "flat"):
        k = g.standard_normal((T, D)).astype(np.float32)
        if mode == "peaked":
            k[517] = 40 * q[0, 1]
        else:
            k[:] = k[0]
        kq, ks = orc.rotate_quant_rows(k, D)
        vq, vs = orc.rotate_quant_rows(v, D)
        kq, vq = kq.reshape(B, Hkv, T, D), vq.reshape(B, Hkv, T, D)
        ks, vs = ks.reshape(B, Hkv, T), vs.reshape(B, Hkv, T)
        dvt = dev.upload(to_blocks(vq, T))
        ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T), np.uint8)
        do = dev.empty((B, Hq, D), np.float32)
        mi.check(mi.lib.mi_gqa_decode_attn_tiled(dev.upload(q).ptr, dev.upload(to_tiles(kq, T)).ptr, dev.upload(ks).ptr, dvt.ptr,
                                              dev.upload(vs).ptr, do.ptr, B, Hq, Hkv, D, T, None, T, 1, ws.ptr, ws.nbytes,
                                              None))
        o = dev.download(do)
        oo = orc.gqa_decode(q, kq, ks, vq, vs, out_rotated=True)
        scale = np.max(np.abs(oo))
        assert np.max(np.abs(o - oo)) <= 2e-6 * max(scale, 1.0), mode
    dev.reset_to(mark)


def test_vt_full_config(mi, dev, orc):
    """cfg2 (B=16, 32/8 heads, T=4096) in this layout: three batch entries against the oracle, every row inside
    the hull of its dequantized V rows, two equal queries of one group give equal rows, and the result agrees with
    the row-major kernel's."""
    mark = dev.mark()
    c = workload.ATTN
    B, Hq, Hkv, T = c["B"], c["Hq"], c["Hkv"], c["T"]
    q, kq, ks, vq, vs, _, _ = make_cache(mi, dev, 2024, B, Hq, Hkv, T, T)
    q[3, 9] = q[3, 8]
    dq, dkq, dks, dvq, dvs = dev.upload(q), dev.upload(kq), dev.upload(ks), dev.upload(vq), dev.upload(vs)
    dkt, dvt = convert(mi, dev, kq, vq, T, T)
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, 128, T), np.uint8)
    do, do2 = dev.empty((B, Hq, 128), np.float32), dev.empty((B, Hq, 128), np.float32)
    mi.check(mi.lib.mi_gqa_decode_attn_tiled(dq.ptr, dkt.ptr, dks.ptr, dvt.ptr, dvs.ptr, do.ptr, B, Hq, Hkv, 128, T, None, T,
                                             1, ws.ptr, ws.nbytes, None))
    o = dev.download(do)
    mi.gqa_decode(dq, dkq, dks, dvq, dvs, do2, True, ws)
    o_rows = dev.download(do2)
    dev.reset_to(mark)
    assert np.array_equal(o[3, 9], o[3, 8])
    assert np.max(np.abs(o - o_rows)) <= 2e-5
    for b in (0, 3, 15):
        oo = orc.gqa_decode(q[b:b + 1], kq[b:b + 1], ks[b:b + 1], vq[b:b + 1], vs[b:b + 1], out_rotated=True)
        assert np.max(np.abs(o[b] - oo[0])) <= 2e-5
    vmax = np.max(np.abs(vq.astype(np.float32)) * vs[..., None], axis=2)
    assert np.all(np.abs(o) <= np.repeat(vmax, Hq // Hkv, axis=1) + 1e-5)


def test_vt_append_matches_row_major_append(mi, dev, orc):
    """The append of this layout writes the codes the row-major append writes, at the transposed place, and touches
    nothing else; with and without the rotary embedding."""
    mark = dev.mark()
    B, Hq, Hkv, T_cap, D = 3, 8, 2, 192, 128
    g = np.random.default_rng(9)
    pos = np.array([0, 100, 191], np.int32)
    NQ = (Hq + 2 * Hkv) * D
    qkv = g.standard_normal((B, NQ)).astype(np.float32)
    ang = g.uniform(0, 6.28, (T_cap, D // 2)).astype(np.float32)
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    dqkv, dcos, dsin, dpos = dev.upload(qkv), dev.upload(cos), dev.upload(sin), dev.upload(pos)

    def fresh():
        junk = np.random.default_rng(2)
        return (dev.upload(junk.integers(-127, 128, (B, Hkv, T_cap, D)).astype(np.int8)),
                dev.upload(junk.random((B, Hkv, T_cap)).astype(np.float32)),
                dev.upload(junk.integers(-127, 128, (B, Hkv, T_cap, D)).astype(np.int8)),
                dev.upload(junk.random((B, Hkv, T_cap)).astype(np.float32)))
    for rope in (False, True):
        kq_a, ks_a, vq_a, vs_a = fresh()
        kq_b, ks_b, vt_b, vs_b = fresh()
        before_v, before_k = dev.download(vq_a), dev.download(kq_a)
        dq_a, dq_b = dev.empty((B, Hq, D), np.float32), dev.empty((B, Hq, D), np.float32)
        if rope:
            mi.check(mi.lib.mi_rope_kv_append_f32_i8(dqkv.ptr, NQ, dcos.ptr, dsin.ptr, dq_a.ptr, kq_a.ptr, ks_a.ptr,
                                                     vq_a.ptr, vs_a.ptr, dpos.ptr, B, Hq, Hkv, D, T_cap, None))
            mi.check(mi.lib.mi_rope_kv_append_tiled_f32_i8(dqkv.ptr, NQ, dcos.ptr, dsin.ptr, dq_b.ptr, kq_b.ptr, ks_b.ptr,
                                                        vt_b.ptr, vs_b.ptr, dpos.ptr, B, Hq, Hkv, D, T_cap, None))
            assert np.array_equal(dev.download(dq_a), dev.download(dq_b))
        else:
            kn, vn = dqkv.ptr + Hq * D * 4, dqkv.ptr + (Hq + Hkv) * D * 4
            mi.check(mi.lib.mi_kv_append_f32_i8(kn, vn, NQ, kq_a.ptr, ks_a.ptr, vq_a.ptr, vs_a.ptr, dpos.ptr, B, Hkv, D,
                                                T_cap, None))
            mi.check(mi.lib.mi_kv_append_tiled_f32_i8(kn, vn, NQ, kq_b.ptr, ks_b.ptr, vt_b.ptr, vs_b.ptr, dpos.ptr, B, Hkv, D,
                                                   T_cap, None))
        # both caches started from the same junk bytes, each in its own order: compare in token-major order
        assert np.array_equal(dev.download(ks_a), dev.download(ks_b))
        assert np.array_equal(dev.download(vs_a), dev.download(vs_b))
        vt = from_blocks(dev.download(vt_b).reshape(B, Hkv, T_cap // 64, D, 64))
        kt = from_tiles(dev.download(kq_b).reshape(B, Hkv, T_cap // 16, 8, 16, 16))
        want_v = from_blocks(before_v.reshape(B, Hkv, T_cap // 64, D, 64)).copy()
        want_k = from_tiles(before_k.reshape(B, Hkv, T_cap // 16, 8, 16, 16)).copy()
        rows_v, rows_k = dev.download(vq_a), dev.download(kq_a)
        for b in range(B):
            want_v[b, :, pos[b]] = rows_v[b, :, pos[b]]
            want_k[b, :, pos[b]] = rows_k[b, :, pos[b]]
        assert np.array_equal(vt, want_v)
        assert np.array_equal(kt, want_k)
    dev.reset_to(mark)


@pytest.mark.parametrize("B,Hq,Hkv,T_cap,N", [(1, 32, 8, 4096, 4096), (1, 16, 4, 1024, 2048), (1, 32, 8, 64, 6144),
                                               (1, 8, 2, 256, 1024), (3, 32, 8, 512, 4096), (16, 32, 8, 256, 4096)])
def test_vt_attention_with_projection_is_the_two_calls(mi, dev, orc, B, Hq, Hkv, T_cap, N):
    """mi_gqa_decode_attn_tiled_linear_f32 = mi_gqa_decode_attn_tiled_quant_i8 + mi_w8a8_gemm_dequant_f32, bit for bit,
    also where it divides the work differently (one token with 2048 or 4096 attention values: merge over many
    workgroups, quantizer inside the projection's GEMV); ragged lengths; the merged row comes back on request."""
    lib = mi.lib
    mark = dev.mark()
    D, K = 128, Hq * 128
    lens = np.array([T_cap, 1, 77, T_cap - 3] * 4, np.int32)[:B]
    q, kq, ks, vq, vs, _, _ = make_cache(mi, dev, 23 + B, B, Hq, Hkv, T_cap, T_cap)
    dkt, dvt = convert(mi, dev, kq, vq, T_cap, T_cap)
    dq, dks, dvs, dl = dev.upload(q), dev.upload(ks), dev.upload(vs), dev.upload(lens)
    w = workload.normal(5, (N, K), 3)
    dqw, dsw = dev.empty((N, K), np.int8), dev.empty(N, np.float32)
    mi.fwht_quant(dev.upload(w), dqw, dsw, 128)
    # the two calls
    ws = dev.empty(lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T_cap), np.uint8)
    orot, oq, osc = dev.empty((B, Hq, D), np.float32), dev.empty((B, K), np.int8), dev.empty(B, np.float32)
    y0 = dev.empty((B, N), np.float32)
    mi.check(lib.mi_gqa_decode_attn_tiled_quant_i8(dq.ptr, dkt.ptr, dks.ptr, dvt.ptr, dvs.ptr, orot.ptr, oq.ptr, osc.ptr, B,
                                                   Hq, Hkv, D, T_cap, dl.ptr, T_cap, ws.ptr, ws.nbytes, None))
    mi.check(lib.mi_w8a8_gemm_dequant_f32(oq.ptr, osc.ptr, dqw.ptr, dsw.ptr, y0.ptr, B, N, K, None))
    # the one call, with and without the merged row
    need = lib.mi_gqa_decode_attn_linear_workspace_bytes(B, Hq, Hkv, D, T_cap)
    assert need > ws.nbytes
    ws2 = dev.upload(np.full(need, 0xA5, np.uint8))
    orot2, y1, y2 = dev.empty((B, Hq, D), np.float32), dev.empty((B, N), np.float32), dev.empty((B, N), np.float32)
    args = (dq.ptr, dkt.ptr, dks.ptr, dvt.ptr, dvs.ptr)
    tail = (B, Hq, Hkv, D, T_cap, dl.ptr, T_cap, N, ws2.ptr, ws2.nbytes, None)
    mi.check(lib.mi_gqa_decode_attn_tiled_linear_f32(*args, orot2.ptr, dqw.ptr, dsw.ptr, y1.ptr, *tail))
    mi.check(lib.mi_gqa_decode_attn_tiled_linear_f32(*args, None, dqw.ptr, dsw.ptr, y2.ptr, *tail))
    a, b, c = dev.download(y0), dev.download(y1), dev.download(y2)
    r0, r1 = dev.download(orot), dev.download(orot2)
    # ... and against the oracle, stage by stage, whatever the division of the work: the merged rows are the
    # oracle's attention (rotated basis) on every sequence's prefix; the codes and the scale the one call left in its
    # workspace are the oracle's quantizer on the device's own merged row; y is the oracle's contraction and
    # dequantization of those codes
    al = lambda n: (n + 255) // 256 * 256
    wsh = dev.download(ws2)
    codes = wsh[al(B * K * 4):al(B * K * 4) + B * K].view(np.int8).reshape(B, K)
    scales = wsh[al(B * K * 4) + al(B * K):al(B * K * 4) + al(B * K) + 4 * B].view(np.float32)
    qw_h, sw_h = dev.download(dqw), dev.download(dsw)
    for s in range(B):
        L = int(lens[s])
        oo = orc.gqa_decode(q[s:s + 1], kq[s:s + 1, :, :L], ks[s:s + 1, :, :L], vq[s:s + 1, :, :L], vs[s:s + 1, :, :L],
                            out_rotated=True)
        assert np.max(np.abs(r1[s] - oo[0])) <= 2e-5, s
        cq, cs = orc.quant_row(r1[s].reshape(-1))
        assert np.array_equal(codes[s], cq) and scales[s] == cs, s
    assert np.array_equal(b, orc.dequant(orc.gemm_i8_i32(codes, qw_h), scales, sw_h))
    assert lib.mi_gqa_decode_attn_tiled_linear_f32(*args, None, dqw.ptr, dsw.ptr, y2.ptr, B, Hq, Hkv, D, T_cap, dl.ptr, T_cap,
                                                   N, ws2.ptr, need - 256, None) == mi.ENOSPC
    dev.reset_to(mark)
    assert np.isfinite(a).all() and np.abs(a).max() > 0
    assert np.array_equal(r0, r1)
    assert np.array_equal(a, b) and np.array_equal(a, c)


# ---- the paged form of the tiled cache, and the gate on the tiled kernel's own integers

def to_pages(dense, table, Hkv, per_page):
    """dense [B, Hkv, nblk, per_page...] -> pool [pages, Hkv, per_page...] under table [B, max_pages] (unused pages: junk)"""
    B, _, nblk = dense.shape[:3]
    pages = int(table.max()) + 1
    pool = np.random.default_rng(5).integers(-100, 100, (pages, Hkv) + dense.shape[3:]).astype(dense.dtype)
    for b in range(B):
        for i in range(nblk):
            if table[b, i] >= 0:
                pool[table[b, i]] = dense[b, :, i]
    return pool


@pytest.mark.parametrize("B,Hq,Hkv,T_cap,lens", [
    (2, 8, 2, 256, [256, 256]), (3, 8, 2, 512, [512, 65, 300]), (4, 16, 4, 1024, [1000, 1, 64, 129]),
    (16, 32, 8, 4096, [4096] * 16),            # the decode-attention configuration at full size
    (1, 32, 8, 2048, [1999]),                  # one sequence: many splits
])
def test_paged_tiled_attention_equals_dense(mi, dev, orc, B, Hq, Hkv, T_cap, lens):
    """The same cache cut into 64-token pages that lie in a shuffled pool: the output equals the dense layout's bit
    for bit (and the oracle within the gate, through the dense test above); table entries behind a sequence's last
    block are poisoned."""
    mark = dev.mark()
    lens = np.array(lens, np.int32)
    q, kq, ks, vq, vs, _, _ = make_cache(mi, dev, 900 + T_cap, B, Hq, Hkv, T_cap, T_cap)
    dkt, dvt = convert(mi, dev, kq, vq, T_cap, T_cap)
    nblk = T_cap // 64
    g = np.random.default_rng(B + T_cap)
    table = g.permutation(B * nblk + 7)[:B * nblk].reshape(B, nblk).astype(np.int32)
    kt_pool = to_pages(dev.download(dkt).reshape(B, Hkv, nblk, 8192), table, Hkv, 8192)
    vt_pool = to_pages(dev.download(dvt).reshape(B, Hkv, nblk, 8192), table, Hkv, 8192)
    ks_pool = to_pages(ks.reshape(B, Hkv, nblk, 64), table, Hkv, 64)
    vs_pool = to_pages(vs.reshape(B, Hkv, nblk, 64), table, Hkv, 64)
    poisoned = table.copy()
    for b in range(B):
        poisoned[b, (int(lens[b]) + 63) // 64:] = 0x3FFFFFF   # never looked up
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, 128, T_cap), np.uint8)
    dq, dks, dvs, dl = dev.upload(q), dev.upload(ks), dev.upload(vs), dev.upload(lens)
    dense_o, paged_o = dev.empty((B, Hq, 128), np.float32), dev.empty((B, Hq, 128), np.float32)
    mi.check(mi.lib.mi_gqa_decode_attn_tiled(dq.ptr, dkt.ptr, dks.ptr, dvt.ptr, dvs.ptr, dense_o.ptr, B, Hq, Hkv, 128, T_cap,
                                             dl.ptr, T_cap, 0, ws.ptr, ws.nbytes, None))
    dev.sync()
    args = (dev.upload(kt_pool), dev.upload(ks_pool), dev.upload(vt_pool), dev.upload(vs_pool))
    mi.check(mi.lib.mi_gqa_decode_attn_tiled_paged(dq.ptr, args[0].ptr, args[1].ptr, args[2].ptr, args[3].ptr, paged_o.ptr,
                                                   dev.upload(poisoned).ptr, nblk, B, Hq, Hkv, 128, dl.ptr, T_cap, 0,
                                                   ws.ptr, ws.nbytes, None), "mi_gqa_decode_attn_tiled_paged")
    od, op = dev.download(dense_o), dev.download(paged_o)
    assert np.array_equal(od, op)
    for b in range(B):   # and the dense result is the oracle's, sequence by sequence
        L = int(lens[b])
        oo = orc.gqa_decode(q[b:b + 1], kq[b:b + 1, :, :L], ks[b:b + 1, :, :L], vq[b:b + 1, :, :L], vs[b:b + 1, :, :L])
        assert np.max(np.abs(op[b:b + 1] - oo)) <= 2e-5
    dev.reset_to(mark)


def test_paged_tiled_append_equals_dense_append(mi, dev):
    """Tokens appended one decode step at a time into a paged pool land exactly where the dense append puts them."""
    mark = dev.mark()
    B, Hkv, T_cap, D = 3, 2, 192, 128
    nblk = T_cap // 64
    g = np.random.default_rng(3)
    table = g.permutation(B * nblk + 3)[:B * nblk].reshape(B, nblk).astype(np.int32)
    pages = int(table.max()) + 1
    dkt, dvt = dev.empty((B, Hkv, nblk, 8192), np.int8), dev.empty((B, Hkv, nblk, 8192), np.int8)
    dks, dvs = dev.empty((B, Hkv, T_cap), np.float32), dev.empty((B, Hkv, T_cap), np.float32)
    pkt, pvt = dev.empty((pages, Hkv, 8192), np.int8), dev.empty((pages, Hkv, 8192), np.int8)
    pks, pvs = dev.empty((pages, Hkv, 64), np.float32), dev.empty((pages, Hkv, 64), np.float32)
    for buf in (dkt, dvt, dks, dvs, pkt, pvt, pks, pvs):
        mi.check(mi.lib.mi_fill_u32(buf.ptr, 0, buf.nbytes // 4, None))
    dtab = dev.upload(table)
    positions = [np.array([0, 63, 64], np.int32), np.array([1, 64, 191], np.int32), np.array([70, 5, 130], np.int32)]
    for step, pos in enumerate(positions):
        k_new = workload.normal(40 + step, (B, Hkv * D), 0)
        v_new = workload.normal(40 + step, (B, Hkv * D), 1)
        dk, dv, dp = dev.upload(k_new), dev.upload(v_new), dev.upload(pos)
        mi.check(mi.lib.mi_kv_append_tiled_f32_i8(dk.ptr, dv.ptr, Hkv * D, dkt.ptr, dks.ptr, dvt.ptr, dvs.ptr, dp.ptr,
                                                  B, Hkv, D, T_cap, None))
        mi.check(mi.lib.mi_kv_append_tiled_paged_f32_i8(dk.ptr, dv.ptr, Hkv * D, pkt.ptr, pks.ptr, pvt.ptr, pvs.ptr,
                                                        dtab.ptr, nblk, dp.ptr, B, Hkv, D, None),
                 "mi_kv_append_tiled_paged_f32_i8")
    dev.sync()
    kt, vt, ks, vs = (dev.download(x) for x in (dkt, dvt, dks, dvs))
    gkt, gvt, gks, gvs = (dev.download(x) for x in (pkt, pvt, pks, pvs))
    for b in range(B):
        for i in range(nblk):
            pg = table[b, i]
            assert np.array_equal(gkt[pg], kt[b, :, i]) and np.array_equal(gvt[pg], vt[b, :, i])
            assert np.array_equal(gks[pg], ks[b, :, 64 * i:64 * i + 64]) and np.array_equal(gvs[pg], vs[b, :, 64 * i:64 * i + 64])
    dev.reset_to(mark)


@pytest.mark.parametrize("B,Hq,Hkv,T,T_cap", [
    (2, 8, 2, 256, 256), (1, 4, 1, 16, 64), (1, 32, 8, 1000, 1024), (3, 6, 3, 77, 128), (1, 8, 2, 4096, 4096),
])
def test_tiled_kernel_scores_are_the_oracles_integers(mi, dev, orc, B, Hq, Hkv, T, T_cap):
    """The tiled kernel's own query codes, query scales and raw int32 dots (the products of its matrix instructions
    on the tiled keys), against the oracle's: bit for bit."""
    mark = dev.mark()
    q, kq, ks, vq, vs, ks_c, vs_c = make_cache(mi, dev, 500 + T, B, Hq, Hkv, T, T_cap)
    dkt, dvt = convert(mi, dev, kq, vq, T, T_cap)
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, 128, T_cap), np.uint8)
    dqq, dsq, ddots = dev.empty((B, Hq, 128), np.int8), dev.empty((B, Hq), np.float32), dev.empty((B, Hq, T), np.int32)
    mi.check(mi.lib.mi_fill_u32(ddots.ptr, 0x7F7F7F7F, ddots.nbytes // 4, None))
    mi.check(mi.lib.mi_gqa_decode_scores_tiled_i32(dev.upload(q).ptr, dkt.ptr, dev.upload(ks_c).ptr, dvt.ptr,
                                                   dev.upload(vs_c).ptr, dqq.ptr, dsq.ptr, ddots.ptr, B, Hq, Hkv, 128,
                                                   T_cap, T, ws.ptr, ws.nbytes, None), "mi_gqa_decode_scores_tiled_i32")
    _, qq, sq, dots = orc.gqa_decode(q, kq, ks, vq, vs, want_debug=True)
    assert np.array_equal(dev.download(dqq), qq)
    assert np.array_equal(dev.download(dsq), sq)
    assert np.array_equal(dev.download(ddots), dots)
    dev.reset_to(mark)


def test_vt_weights_with_v_scales_over_six_decades(mi, dev, orc):
    """The fixed-point weights are relative to the largest V scale of a split.  Here the V scales spread over six
    decades and the softmax mass sits on the tokens with the SMALLEST scales (their keys are the query scaled up),
    so their weights keep only about 28 - 20 bits: the output must stay inside the bound the header states,
    T * 127 * 2^-29 * vmax, and, the roundings being to nearest, well inside it (1 % of the output's size)."""
    mark = dev.mark()
    B, Hq, Hkv, T, D = 1, 4, 1, 1024, 128
    g = np.random.default_rng(15)
    q = g.standard_normal((B, Hq, D)).astype(np.float32)
    q[0, 1:] = q[0, 0]                               # one direction, so that the same tokens win for every head
    mag = np.exp(g.uniform(-7.0, 7.0, (T, 1)))
    v = (g.standard_normal((T, D)) * mag).astype(np.float32)
    k = g.standard_normal((T, D)).astype(np.float32)
    small = np.argsort(mag[:, 0])[:48]
    k[small] = 3.0 * q[0, 0]
    kq, ks = orc.rotate_quant_rows(k, D)
    vq, vs = orc.rotate_quant_rows(v, D)
    kq, vq = kq.reshape(B, Hkv, T, D), vq.reshape(B, Hkv, T, D)
    ks, vs = ks.reshape(B, Hkv, T), vs.reshape(B, Hkv, T)
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T), np.uint8)
    do = dev.empty((B, Hq, D), np.float32)
    mi.check(mi.lib.mi_gqa_decode_attn_tiled(dev.upload(q).ptr, dev.upload(to_tiles(kq, T)).ptr, dev.upload(ks).ptr,
                                             dev.upload(to_blocks(vq, T)).ptr, dev.upload(vs).ptr, do.ptr, B, Hq, Hkv, D,
                                             T, None, T, 1, ws.ptr, ws.nbytes, None))
    o = dev.download(do)
    oo = orc.gqa_decode(q, kq, ks, vq, vs, out_rotated=True)
    size = float(np.max(np.abs(oo)))
    assert size < 1e-3 * float(vs.max()) * 127          # the mass really is on the small-scale tokens
    err = float(np.max(np.abs(o - oo)))
    assert err <= T * 127 * 2.0 ** -29 * float(vs.max())
    assert err <= 1e-2 * size, (err, size)
    dev.reset_to(mark)
