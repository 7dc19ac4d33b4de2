"""GPU parity: the KV-cache append path and attention over a partly filled cache.
Gates: appended codes and scales bit-exact against the oracle quantizer, every other cache entry untouched;
attention per sequence max-abs <= 2e-3 against the oracle run on that sequence's own prefix."""
import numpy as np
import pytest

import workload

pytestmark = pytest.mark.gpu

TOL = 2e-3
D = 128


def alloc_cache(dev, B, Hkv, T_cap):
    return (dev.empty((B, Hkv, T_cap, D), np.int8), dev.empty((B, Hkv, T_cap), np.float32),
            dev.empty((B, Hkv, T_cap, D), np.int8), dev.empty((B, Hkv, T_cap), np.float32))


def append(mi, dk, dv, row_stride, cache, dpos, B, Hkv, T_cap):
    dkq, dks, dvq, dvs = cache
    mi.check(mi.lib.mi_kv_append_f32_i8(dk, dv, row_stride, dkq.ptr, dks.ptr, dvq.ptr, dvs.ptr, dpos.ptr,
                                        B, Hkv, D, T_cap, None), "mi_kv_append_f32_i8")


@pytest.mark.parametrize("B,Hkv,T_cap", [(3, 2, 40), (16, 8, 64), (1, 1, 1), (5, 3, 17)])
def test_append_writes_oracle_codes_at_positions_only(mi, dev, orc, B, Hkv, T_cap):
    mark = dev.mark()
    g = np.random.default_rng(B * 100 + T_cap)
    cache = alloc_cache(dev, B, Hkv, T_cap)
    # recognisable background so that stray writes show
    bg_q = g.integers(-127, 128, (B, Hkv, T_cap, D)).astype(np.int8)
    bg_s = g.random((B, Hkv, T_cap), dtype=np.float32)
    for buf, bg in zip(cache, (bg_q, bg_s, bg_q, bg_s)):
        mi.check(mi.lib.mi_memcpy_h2d(buf.ptr, bg.ctypes.data, bg.nbytes, None))
    k = workload.normal(3, (B, Hkv, D), 1)
    v = workload.normal(3, (B, Hkv, D), 2)
    k[0, 0] = 0.0                                        # an all-zero head: scale 1, codes 0
    pos = g.integers(0, T_cap, B).astype(np.int32)
    if B > 2:
        pos[1] = T_cap                                   # outside the cache: skipped
        pos[2] = -1
    dk, dv, dpos = dev.upload(k), dev.upload(v), dev.upload(pos)
    append(mi, dk.ptr, dv.ptr, Hkv * D, cache, dpos, B, Hkv, T_cap)
    kq, ks, vq, vs = (dev.download(b) for b in cache)
    dev.reset_to(mark)
    want_kq, want_ks, want_vq, want_vs = bg_q.copy(), bg_s.copy(), bg_q.copy(), bg_s.copy()
    kqo, kso = orc.rotate_quant_rows(k.reshape(-1, D), D)
    vqo, vso = orc.rotate_quant_rows(v.reshape(-1, D), D)
    for b in range(B):
        if 0 <= pos[b] < T_cap:
            for h in range(Hkv):
                want_kq[b, h, pos[b]] = kqo[b * Hkv + h]; want_ks[b, h, pos[b]] = kso[b * Hkv + h]
                want_vq[b, h, pos[b]] = vqo[b * Hkv + h]; want_vs[b, h, pos[b]] = vso[b * Hkv + h]
    assert np.array_equal(kq, want_kq) and np.array_equal(ks, want_ks)
    assert np.array_equal(vq, want_vq) and np.array_equal(vs, want_vs)
    assert ks[0, 0, pos[0]] == 1.0 and not kq[0, 0, pos[0]].any()


def test_append_reads_slices_of_a_fused_qkv_row(mi, dev, orc):
    """k and v taken in place from rows [q | k | v] of a projection output."""
    mark = dev.mark()
    B, Hq, Hkv, T_cap = 4, 8, 2, 8
    row = (Hq + 2 * Hkv) * D
    qkv = workload.normal(11, (B, row), 0)
    dqkv = dev.upload(qkv)
    cache = alloc_cache(dev, B, Hkv, T_cap)
    pos = np.array([0, 3, 7, 5], np.int32)
    dpos = dev.upload(pos)
    append(mi, dqkv.ptr + 4 * Hq * D, dqkv.ptr + 4 * (Hq + Hkv) * D, row, cache, dpos, B, Hkv, T_cap)
    kq, ks, vq, vs = (dev.download(b) for b in cache)
    dev.reset_to(mark)
    k = qkv[:, Hq * D:(Hq + Hkv) * D].reshape(B * Hkv, D)
    v = qkv[:, (Hq + Hkv) * D:].reshape(B * Hkv, D)
    kqo, kso = orc.rotate_quant_rows(np.ascontiguousarray(k), D)
    vqo, vso = orc.rotate_quant_rows(np.ascontiguousarray(v), D)
    for b in range(B):
        for h in range(Hkv):
            assert np.array_equal(kq[b, h, pos[b]], kqo[b * Hkv + h]) and ks[b, h, pos[b]] == kso[b * Hkv + h]
            assert np.array_equal(vq[b, h, pos[b]], vqo[b * Hkv + h]) and vs[b, h, pos[b]] == vso[b * Hkv + h]


def cache_attention(mi, dev, dq, cache, dlen, B, Hq, Hkv, T_cap, T_max, out_rotated):
    dkq, dks, dvq, dvs = cache
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T_max), np.uint8)
    do = dev.empty((B, Hq, D), np.float32)
    mi.check(mi.lib.mi_gqa_decode_attn_cache(dq.ptr, dkq.ptr, dks.ptr, dvq.ptr, dvs.ptr, do.ptr, B, Hq, Hkv, D,
                                             T_cap, dlen.ptr, T_max, 1 if out_rotated else 0, ws.ptr, ws.nbytes,
                                             None), "mi_gqa_decode_attn_cache")
    return dev.download(do)


def oracle_per_sequence(orc, q, kq, ks, vq, vs, lens, out_rotated):
    out = np.zeros_like(q)
    for b, n in enumerate(lens):
        if n > 0:
            out[b] = orc.gqa_decode(q[b:b + 1], np.ascontiguousarray(kq[b:b + 1, :, :n]),
                                    np.ascontiguousarray(ks[b:b + 1, :, :n]),
                                    np.ascontiguousarray(vq[b:b + 1, :, :n]),
                                    np.ascontiguousarray(vs[b:b + 1, :, :n]), out_rotated=out_rotated)[0]
    return out


@pytest.mark.parametrize("B,Hq,Hkv,T_cap,lens", [
    (4, 8, 2, 1024, [1, 700, 1024, 333]),          # several splits, some of them past the end of a sequence
    (3, 4, 1, 100, [100, 17, 64]),
    (2, 32, 8, 4096, [4096, 2500]),
    (3, 6, 3, 48, [0, 5, 48]),                     # an empty sequence gives zeros
])
@pytest.mark.parametrize("out_rotated", [False, True])
def test_attention_over_partly_filled_cache(mi, dev, orc, B, Hq, Hkv, T_cap, lens, out_rotated):
    mark = dev.mark()
    g = np.random.default_rng(T_cap + B)
    q = workload.normal(T_cap, (B, Hq, D), 0)
    kq = g.integers(-127, 128, (B, Hkv, T_cap, D)).astype(np.int8)
    vq = g.integers(-127, 128, (B, Hkv, T_cap, D)).astype(np.int8)
    ks = (g.random((B, Hkv, T_cap), dtype=np.float32) + 0.5) * np.float32(0.02)
    vs = (g.random((B, Hkv, T_cap), dtype=np.float32) + 0.5) * np.float32(0.02)
    lens = np.array(lens, np.int32)
    # entries past a sequence's length hold values that would wreck the result if they were read into it
    for b, n in enumerate(lens):
        ks[b, :, n:] = np.float32(1e30)
        vs[b, :, n:] = np.float32(np.nan)
    cache = tuple(dev.upload(a) for a in (kq, ks, vq, vs))
    dq, dlen = dev.upload(q), dev.upload(lens)
    T_max = int(max(lens.max(), 1))
    o = cache_attention(mi, dev, dq, cache, dlen, B, Hq, Hkv, T_cap, T_max, out_rotated)
    o_cap = cache_attention(mi, dev, dq, cache, dlen, B, Hq, Hkv, T_cap, T_cap, out_rotated)   # looser bound, more splits
    dev.reset_to(mark)
    want = oracle_per_sequence(orc, q, kq, ks, vq, vs, lens, out_rotated)
    assert np.isfinite(o).all() and np.isfinite(o_cap).all()
    assert np.max(np.abs(o - want)) <= 2e-5 and np.max(np.abs(o_cap - want)) <= 2e-5   # gate: TOL
    assert np.max(np.abs(o - want)) <= TOL


@pytest.mark.parametrize("B,Hq,Hkv,T_cap,lens", [(4, 32, 8, 1024, [1, 700, 1024, 333]), (2, 8, 8, 64, [64, 0]),
                                                  (3, 64, 16, 40, [40, 7, 22])])
def test_attention_merge_fused_with_the_output_quantizer(mi, dev, orc, B, Hq, Hkv, T_cap, lens):
    """The fused entry leaves the same rotated-basis rows as the plain one (same merge arithmetic) and their codes
    and scale are the oracle's row quantizer applied to each token's Hq*128 values."""
    mark = dev.mark()
    g = np.random.default_rng(T_cap)
    q = workload.normal(T_cap + 1, (B, Hq, D), 0)
    kq = g.integers(-127, 128, (B, Hkv, T_cap, D)).astype(np.int8)
    vq = g.integers(-127, 128, (B, Hkv, T_cap, D)).astype(np.int8)
    ks = ((g.random((B, Hkv, T_cap)) + 0.5) * 0.02).astype(np.float32)
    vs = ((g.random((B, Hkv, T_cap)) + 0.5) * 0.02).astype(np.float32)
    lens = np.array(lens, np.int32)
    cache = tuple(dev.upload(a) for a in (kq, ks, vq, vs))
    dq, dlen = dev.upload(q), dev.upload(lens)
    T_max = int(max(lens.max(), 1))
    plain = cache_attention(mi, dev, dq, cache, dlen, B, Hq, Hkv, T_cap, T_max, True)
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T_max), np.uint8)
    do, doq, dos = dev.empty((B, Hq, D), np.float32), dev.empty((B, Hq * D), np.int8), dev.empty(B, np.float32)
    args = (dq.ptr, cache[0].ptr, cache[1].ptr, cache[2].ptr, cache[3].ptr)
    tail = (B, Hq, Hkv, D, T_cap, dlen.ptr, T_max, ws.ptr, ws.nbytes, None)
    mi.check(mi.lib.mi_gqa_decode_attn_cache_quant_i8(*args, do.ptr, doq.ptr, dos.ptr, *tail))
    o, oq, osc = dev.download(do), dev.download(doq), dev.download(dos)
    mi.check(mi.lib.mi_gqa_decode_attn_cache_quant_i8(*args, None, doq.ptr, dos.ptr, *tail))     # without the fp32 row
    oq2, osc2 = dev.download(doq), dev.download(dos)
    assert mi.lib.mi_gqa_decode_attn_cache_quant_i8(*args, None, None, dos.ptr, *tail) == mi.EINVAL
    dev.reset_to(mark)
    assert np.array_equal(o, plain)
    for b in range(B):
        qo, so = orc.quant_row(o[b].reshape(-1))
        assert np.array_equal(oq[b], qo) and osc[b] == so
    assert np.array_equal(oq, oq2) and np.array_equal(osc, osc2)
    assert not o[lens == 0].any() and np.all(osc[lens == 0] == 1.0)


def test_decode_loop_append_then_attend(mi, dev, orc):
    """Six decode steps on sequences of different lengths: each step appends one token per sequence at its own
    position and attends over what the sequence holds so far; the cache and every output follow the oracle."""
    mark = dev.mark()
    B, Hq, Hkv, T_cap, steps = 3, 8, 2, 96, 6
    start = np.array([0, 40, 89], np.int32)          # the third sequence reaches the end of the cache
    cache = alloc_cache(dev, B, Hkv, T_cap)
    ref_kq = np.zeros((B, Hkv, T_cap, D), np.int8); ref_ks = np.zeros((B, Hkv, T_cap), np.float32)
    ref_vq = np.zeros_like(ref_kq); ref_vs = np.zeros_like(ref_ks)
    # prefixes written through the plain quantizer entry point (same arithmetic)
    for b in range(B):
        n = int(start[b])
        if n == 0:
            continue
        for h in range(Hkv):
            kk = workload.normal(50 + b, (n, D), h)
            vv = workload.normal(60 + b, (n, D), h)
            ref_kq[b, h, :n], ref_ks[b, h, :n] = orc.rotate_quant_rows(kk, D)
            ref_vq[b, h, :n], ref_vs[b, h, :n] = orc.rotate_quant_rows(vv, D)
    for buf, ref in zip(cache, (ref_kq, ref_ks, ref_vq, ref_vs)):
        mi.check(mi.lib.mi_memcpy_h2d(buf.ptr, ref.ctypes.data, ref.nbytes, None))
    dpos, dlen = dev.empty(B, np.int32), dev.empty(B, np.int32)
    for step in range(steps):
        pos = start + step
        k = workload.normal(200 + step, (B, Hkv, D), 1)
        v = workload.normal(200 + step, (B, Hkv, D), 2)
        q = workload.normal(200 + step, (B, Hq, D), 3)
        mi.check(mi.lib.mi_memcpy_h2d(dpos.ptr, pos.ctypes.data, pos.nbytes, None))
        lens = np.minimum(pos + 1, T_cap).astype(np.int32)
        mi.check(mi.lib.mi_memcpy_h2d(dlen.ptr, lens.ctypes.data, lens.nbytes, None))
        m2 = dev.mark()
        dk, dv, dq = dev.upload(k), dev.upload(v), dev.upload(q)
        append(mi, dk.ptr, dv.ptr, Hkv * D, cache, dpos, B, Hkv, T_cap)
        o = cache_attention(mi, dev, dq, cache, dlen, B, Hq, Hkv, T_cap, int(lens.max()), False)
        dev.reset_to(m2)
        kqo, kso = orc.rotate_quant_rows(k.reshape(-1, D), D)
        vqo, vso = orc.rotate_quant_rows(v.reshape(-1, D), D)
        for b in range(B):
            if pos[b] < T_cap:
                ref_kq[b, :, pos[b]] = kqo.reshape(B, Hkv, D)[b]; ref_ks[b, :, pos[b]] = kso.reshape(B, Hkv)[b]
                ref_vq[b, :, pos[b]] = vqo.reshape(B, Hkv, D)[b]; ref_vs[b, :, pos[b]] = vso.reshape(B, Hkv)[b]
        want = oracle_per_sequence(orc, q, ref_kq, ref_ks, ref_vq, ref_vs, lens, False)
        assert np.max(np.abs(o - want)) <= 2e-5, "step %d" % step
    got = [dev.download(b) for b in cache]
    dev.reset_to(mark)
    for a, r in zip(got, (ref_kq, ref_ks, ref_vq, ref_vs)):
        assert np.array_equal(a, r)


def test_bad_arguments_are_refused(mi, dev):
    mark = dev.mark()
    B, Hq, Hkv, T_cap = 2, 4, 2, 16
    cache = alloc_cache(dev, B, Hkv, T_cap)
    x = dev.empty((B, Hkv, D), np.float32)
    pos = dev.empty(B, np.int32)
    lib = mi.lib
    a = (cache[0].ptr, cache[1].ptr, cache[2].ptr, cache[3].ptr, pos.ptr)
    assert lib.mi_kv_append_f32_i8(x.ptr, x.ptr, Hkv * D - 4, *a, B, Hkv, D, T_cap, None) == mi.EINVAL   # rows overlap
    assert lib.mi_kv_append_f32_i8(x.ptr, x.ptr, Hkv * D, *a, B, Hkv, 64, T_cap, None) == mi.EINVAL      # head_dim
    assert lib.mi_kv_append_f32_i8(None, x.ptr, Hkv * D, *a, B, Hkv, D, T_cap, None) == mi.EINVAL
    q = dev.empty((B, Hq, D), np.float32)
    ws = dev.empty(lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T_cap), np.uint8)
    args = (q.ptr, cache[0].ptr, cache[1].ptr, cache[2].ptr, cache[3].ptr, q.ptr, B, Hq, Hkv, D)
    assert lib.mi_gqa_decode_attn_cache(*args, T_cap, pos.ptr, T_cap + 1, 0, ws.ptr, ws.nbytes, None) == mi.EINVAL
    assert lib.mi_gqa_decode_attn_cache(*args, T_cap, None, T_cap, 0, ws.ptr, ws.nbytes, None) == mi.EINVAL
    assert lib.mi_gqa_decode_attn_cache(*args, T_cap, pos.ptr, T_cap, 0, ws.ptr, 16, None) == mi.ENOSPC
    dev.reset_to(mark)


def to_pages(g, dense, P, max_pages, spare=3):
    """Scatter dense cache arrays [B,Hkv,T,...] into pools [pages,Hkv,P,...] under a random block table."""
    B, Hkv, T = dense[0].shape[:3]
    npages = B * max_pages + spare
    table = g.permutation(npages)[:B * max_pages].astype(np.int32).reshape(B, max_pages)
    pools = []
    for a in dense:
        pool = np.zeros((npages, Hkv, P) + a.shape[3:], a.dtype)
        if a.dtype == np.float32:
            pool[...] = np.float32(np.nan)            # a page that is not in the table must never be read
        for b in range(B):
            for i in range(max_pages):
                lo, hi = i * P, min((i + 1) * P, T)
                if lo < T:
                    pool[table[b, i], :, :hi - lo] = a[b, :, lo:hi]
        pools.append(pool)
    return pools, table


@pytest.mark.parametrize("B,Hq,Hkv,T,P,lens", [
    (4, 8, 2, 1024, 16, [1, 700, 1024, 333]),
    (2, 32, 8, 4096, 256, [4096, 2500]),
    (3, 4, 1, 200, 64, [200, 17, 64]),
    (2, 8, 4, 96, 32, [0, 96]),
])
@pytest.mark.parametrize("out_rotated", [False, True])
def test_paged_attention_equals_dense(mi, dev, orc, B, Hq, Hkv, T, P, lens, out_rotated):
    mark = dev.mark()
    g = np.random.default_rng(T + P)
    q = workload.normal(T + P, (B, Hq, D), 0)
    dense = [g.integers(-127, 128, (B, Hkv, T, D)).astype(np.int8), ((g.random((B, Hkv, T)) + 0.5) * 0.02).astype(np.float32),
             g.integers(-127, 128, (B, Hkv, T, D)).astype(np.int8), ((g.random((B, Hkv, T)) + 0.5) * 0.02).astype(np.float32)]
    lens = np.array(lens, np.int32)
    max_pages = (T + P - 1) // P
    pools, table = to_pages(g, dense, P, max_pages)
    # tokens past a sequence's length: poison in the pools as well (same page, later offset)
    cache = tuple(dev.upload(a) for a in dense)
    dpools = tuple(dev.upload(a) for a in pools)
    dq, dlen, dtab = dev.upload(q), dev.upload(lens), dev.upload(table)
    T_max = int(max(lens.max(), 1))
    want_gpu = cache_attention(mi, dev, dq, cache, dlen, B, Hq, Hkv, T, T_max, out_rotated)
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T_max), np.uint8)
    do = dev.empty((B, Hq, D), np.float32)
    mi.check(mi.lib.mi_gqa_decode_attn_paged(dq.ptr, dpools[0].ptr, dpools[1].ptr, dpools[2].ptr, dpools[3].ptr, do.ptr,
                                             dtab.ptr, max_pages, P, B, Hq, Hkv, D, dlen.ptr, T_max,
                                             1 if out_rotated else 0, ws.ptr, ws.nbytes, None),
             "mi_gqa_decode_attn_paged")
    o = dev.download(do)
    dev.reset_to(mark)
    assert np.isfinite(o).all()
    assert np.array_equal(o, want_gpu)                          # same arithmetic in the same order
    want = oracle_per_sequence(orc, q, *dense, lens, out_rotated)
    assert np.max(np.abs(o - want)) <= 2e-5                     # gate: TOL


def test_paged_append_lands_in_the_right_page(mi, dev, orc):
    mark = dev.mark()
    B, Hkv, P, max_pages = 5, 2, 16, 4
    g = np.random.default_rng(77)
    npages = B * max_pages + 2
    table = g.permutation(npages)[:B * max_pages].astype(np.int32).reshape(B, max_pages)
    bgq = g.integers(-127, 128, (npages, Hkv, P, D)).astype(np.int8)
    bgs = g.random((npages, Hkv, P), dtype=np.float32)
    pools = [dev.upload(bgq), dev.upload(bgs), dev.upload(bgq), dev.upload(bgs)]
    k = workload.normal(5, (B, Hkv, D), 1)
    v = workload.normal(5, (B, Hkv, D), 2)
    pos = np.array([0, 15, 16, 63, 64], np.int32)              # the last one is past the table: skipped
    dk, dv, dpos, dtab = dev.upload(k), dev.upload(v), dev.upload(pos), dev.upload(table)
    mi.check(mi.lib.mi_kv_append_paged_f32_i8(dk.ptr, dv.ptr, Hkv * D, pools[0].ptr, pools[1].ptr, pools[2].ptr,
                                              pools[3].ptr, dtab.ptr, max_pages, P, dpos.ptr, B, Hkv, D, None),
             "mi_kv_append_paged_f32_i8")
    kq, ks, vq, vs = (dev.download(b) for b in pools)
    assert mi.lib.mi_kv_append_paged_f32_i8(dk.ptr, dv.ptr, Hkv * D, pools[0].ptr, pools[1].ptr, pools[2].ptr,
                                            pools[3].ptr, dtab.ptr, max_pages, 24, dpos.ptr, B, Hkv, D, None) == mi.EINVAL
    dev.reset_to(mark)
    wkq, wks, wvq, wvs = bgq.copy(), bgs.copy(), bgq.copy(), bgs.copy()
    kqo, kso = orc.rotate_quant_rows(k.reshape(-1, D), D)
    vqo, vso = orc.rotate_quant_rows(v.reshape(-1, D), D)
    for b in range(B):
        if pos[b] < max_pages * P:
            pg, off = table[b, pos[b] // P], pos[b] % P
            for h in range(Hkv):
                wkq[pg, h, off], wks[pg, h, off] = kqo[b * Hkv + h], kso[b * Hkv + h]
                wvq[pg, h, off], wvs[pg, h, off] = vqo[b * Hkv + h], vso[b * Hkv + h]
    assert np.array_equal(kq, wkq) and np.array_equal(ks, wks)
    assert np.array_equal(vq, wvq) and np.array_equal(vs, wvs)
