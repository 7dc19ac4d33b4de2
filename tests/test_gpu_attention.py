"""GPU parity: GQA decode attention over an int8 KV cache.
Gates: query codes and int32 scores bit-exact; output max-abs <= 2e-3."""
import numpy as np
import pytest

import workload

pytestmark = pytest.mark.gpu

TOL = 2e-3


def make_case(mi, dev, orc, seed, B, Hq, Hkv, T, D=128):
    q = workload.normal(seed, (B, Hq, D), 0)
    k = workload.normal(seed, (B * Hkv * T, D), 1)
    v = workload.normal(seed, (B * Hkv * T, D), 2)
    # the KV cache is produced by the GPU quantizer (a7) and gated against the oracle
    dk, dv = dev.upload(k), dev.upload(v)
    dkq, dks = dev.empty((B, Hkv, T, D), np.int8), dev.empty((B, Hkv, T), np.float32)
    dvq, dvs = dev.empty((B, Hkv, T, D), np.int8), dev.empty((B, Hkv, T), np.float32)
    mi.check(mi.lib.mi_fwht_quant_f32_i8(dk.ptr, dkq.ptr, dks.ptr, B * Hkv * T, D, D, None))
    mi.check(mi.lib.mi_fwht_quant_f32_i8(dv.ptr, dvq.ptr, dvs.ptr, B * Hkv * T, D, D, None))
    return q, k, v, dev.upload(q), dkq, dks, dvq, dvs


@pytest.mark.parametrize("B,Hq,Hkv,T", [
    (2, 8, 2, 256), (1, 4, 1, 16), (1, 32, 8, 1000), (3, 6, 3, 77), (2, 4, 4, 130), (1, 8, 2, 1),
    (1, 8, 2, 4096),
])
@pytest.mark.parametrize("out_rotated", [False, True])
def test_attention_matches_oracle(mi, dev, orc, B, Hq, Hkv, T, out_rotated):
    mark = dev.mark()
    q, k, v, dq, dkq, dks, dvq, dvs = make_case(mi, dev, orc, 100 + T, B, Hq, Hkv, T)
    kq, ks, vq, vs = (dev.download(b) for b in (dkq, dks, dvq, dvs))
    kqo, kso = orc.rotate_quant_rows(k, 128)
    assert np.array_equal(kq.reshape(-1, 128), kqo) and np.array_equal(ks.reshape(-1), kso)
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, 128, T), np.uint8)
    do = dev.empty((B, Hq, 128), np.float32)
    mi.gqa_decode(dq, dkq, dks, dvq, dvs, do, out_rotated, ws)
    o = dev.download(do)
    dqq, dsq = dev.empty((B, Hq, 128), np.int8), dev.empty((B, Hq), np.float32)
    ddots = dev.empty((B, Hq, T), np.int32)
    mi.gqa_scores(dq, dkq, dks, dvq, dvs, dqq, dsq, ddots, ws)
    qq, sq, dots = dev.download(dqq), dev.download(dsq), dev.download(ddots)
    dev.reset_to(mark)
    oo, qqo, sqo, dotso = orc.gqa_decode(q, kq, ks, vq, vs, out_rotated=out_rotated, want_debug=True)
    assert np.array_equal(qq, qqo) and np.array_equal(sq, sqo)
    assert np.array_equal(dots, dotso)
    assert np.max(np.abs(o - oo)) <= TOL
    assert np.max(np.abs(o - oo)) <= 2e-5     # fp32 accumulation is far inside the gate


def test_single_token_returns_dequantized_v(mi, dev, orc):
    mark = dev.mark()
    B, Hq, Hkv, T = 2, 8, 2, 1
    q, k, v, dq, dkq, dks, dvq, dvs = make_case(mi, dev, orc, 7, B, Hq, Hkv, T)
    vq, vs = dev.download(dvq), dev.download(dvs)
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, 128, T), np.uint8)
    do = dev.empty((B, Hq, 128), np.float32)
    mi.gqa_decode(dq, dkq, dks, dvq, dvs, do, True, ws)
    o = dev.download(do)
    dev.reset_to(mark)
    for b in range(B):
        for h in range(Hq):
            want = vs[b, h // 4, 0] * vq[b, h // 4, 0].astype(np.float32)
            assert np.max(np.abs(o[b, h] - want)) <= 1e-5


def test_full_config_properties(mi, dev, orc):
    """cfg2: B=16, 32/8 heads, T=4096.  Two (b, kv-head) groups against the
    oracle; every output row must lie inside the convex hull bound of its
    dequantized V rows and heads of one group sharing a query must agree."""
    mark = dev.mark()
    c = workload.ATTN
    B, Hq, Hkv, T = c["B"], c["Hq"], c["Hkv"], c["T"]
    q, k, v, dq, dkq, dks, dvq, dvs = make_case(mi, dev, orc, 2024, B, Hq, Hkv, T)
    q[3, 9] = q[3, 8]                          # same KV group (heads 8..11)
    dq = dev.upload(q)
    ws = dev.empty(mi.lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, 128, T), np.uint8)
    do = dev.empty((B, Hq, 128), np.float32)
    mi.gqa_decode(dq, dkq, dks, dvq, dvs, do, True, ws)
    o = dev.download(do)
    kq, ks, vq, vs = (dev.download(b) for b in (dkq, dks, dvq, dvs))
    dev.reset_to(mark)
    assert np.array_equal(o[3, 9], o[3, 8])
    for b in (0, 3, 15):
        oo = orc.gqa_decode(q[b:b + 1], kq[b:b + 1], ks[b:b + 1], vq[b:b + 1], vs[b:b + 1], out_rotated=True)
        assert np.max(np.abs(o[b] - oo[0])) <= TOL
    vmax = np.max(np.abs(vq.astype(np.float32)) * vs[..., None], axis=2)       # [B,Hkv,D]
    assert np.all(np.abs(o) <= np.repeat(vmax, Hq // Hkv, axis=1) + 1e-5)
    assert np.all(np.isfinite(o))


def test_argument_errors(mi, dev):
    lib = mi.lib
    mark = dev.mark()
    b = dev.empty(1 << 16, np.uint8)
    args = (b.ptr,) * 6
    assert lib.mi_gqa_decode_attn(*args, 1, 8, 2, 64, 16, 0, b.ptr, b.nbytes, None) == mi.EINVAL    # D
    assert lib.mi_gqa_decode_attn(*args, 1, 8, 3, 128, 16, 0, b.ptr, b.nbytes, None) == mi.EINVAL   # Hq % Hkv
    assert lib.mi_gqa_decode_attn(*args, 1, 8, 1, 128, 16, 0, b.ptr, b.nbytes, None) == mi.EINVAL   # group > 4
    assert lib.mi_gqa_decode_attn(*args, 1, 8, 2, 128, 16, 0, b.ptr, 16, None) == mi.ENOSPC
    assert lib.mi_gqa_decode_attn(*args, 1, 8, 2, 128, 0, 0, b.ptr, b.nbytes, None) == mi.EINVAL    # T
    dev.reset_to(mark)
