"""Pins oracle a9 (router), a10 (dispatch) and a11 (grouped expert FFN)."""
import numpy as np
import pytest


def fma32(a, b, c):
    # exact product in float64 (24+24 bits), one float64 add, then to fp32
    return np.float32(np.float64(a) * np.float64(b) + np.float64(c))


def router_dot_python(x, w):
    H = x.size
    part = [np.float32(0)] * 64
    for j in range(H // 256):
        for l in range(64):
            for c in range(4):
                k = 256 * j + 4 * l + c
                part[l] = fma32(x[k], w[k], part[l])
    off = 32
    while off >= 1:
        part = [np.float32(part[l] + part[l ^ off]) for l in range(64)]
        off //= 2
    return part[0]


def test_router_dot_order(orc):
    g = np.random.default_rng(31)
    for H in (256, 2048):
        x = g.standard_normal(H).astype(np.float32)
        w = (g.standard_normal(H) * 0.02).astype(np.float32)
        got = orc.router_dot(x, w)
        assert got == router_dot_python(x, w)
        assert abs(float(got) - float(x.astype(np.float64) @ w.astype(np.float64))) < 1e-5


def test_route_topk_vs_argsort_and_softmax(orc):
    g = np.random.default_rng(32)
    T, H, E, k = 9, 512, 16, 4
    x = g.standard_normal((T, H)).astype(np.float32)
    wr = (g.standard_normal((E, H)) * 0.02).astype(np.float32)
    idx, w, lg = orc.moe_route(x, wr, k, want_logits=True)
    for t in range(T):
        for e in range(E):
            assert lg[t, e] == orc.router_dot(x[t], wr[e])
        order = np.argsort(-lg[t].astype(np.float64), kind="stable")[:k]
        assert idx[t].tolist() == order.tolist()
        p = np.exp(lg[t].astype(np.float64) - lg[t].max())
        p /= p.sum()
        want = p[order] / p[order].sum()       # full softmax, pick, renormalize
        assert np.max(np.abs(w[t] - want)) < 1e-6
        assert abs(float(w[t].sum()) - 1) < 1e-6
        assert np.all(np.diff(w[t]) <= 0)


def test_route_ties_go_to_lower_index(orc):
    g = np.random.default_rng(33)
    H, E, k = 256, 8, 3
    x = g.standard_normal((2, H)).astype(np.float32)
    base = (g.standard_normal((E, H)) * 0.02).astype(np.float32)
    base[5] = base[2]           # exact tie between experts 2 and 5
    base[7] = base[2]
    idx, w, lg = orc.moe_route(x, base, k, want_logits=True)
    for t in range(2):
        assert lg[t, 2] == lg[t, 5] == lg[t, 7]
        picks = idx[t].tolist()
        tied = [e for e in picks if e in (2, 5, 7)]
        assert tied == sorted(tied)
        if 5 in picks:
            assert 2 in picks
        if 7 in picks:
            assert 2 in picks and 5 in picks
    # all experts identical: picks are 0,1,2 with equal weights
    same = np.repeat(base[:1], E, 0)
    idx, w = orc.moe_route(x, same, k)
    assert idx.tolist() == [[0, 1, 2]] * 2
    assert np.allclose(w, 1.0 / 3.0, atol=1e-7)


def test_route_rejects_bad_shapes(orc):
    with pytest.raises(ValueError):
        orc.moe_route(np.zeros((1, 100), np.float32), np.zeros((4, 100), np.float32), 2)
    with pytest.raises(ValueError):
        orc.moe_route(np.zeros((1, 256), np.float32), np.zeros((4, 256), np.float32), 5)


def test_dispatch_is_stable_counting_sort(orc):
    g = np.random.default_rng(34)
    T, k, E = 512, 8, 128
    idx = np.stack([g.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    perm, seg = orc.moe_dispatch(idx, E)
    flat = idx.reshape(-1)
    assert np.array_equal(perm, np.argsort(flat, kind="stable").astype(np.int32))
    assert np.array_equal(seg, np.concatenate([[0], np.cumsum(np.bincount(flat, minlength=E))]))
    assert seg[E] == T * k and sorted(perm.tolist()) == list(range(T * k))


def test_dispatch_empty_experts_and_bad_index(orc):
    idx = np.array([[3, 1], [3, 0]], np.int32)
    perm, seg = orc.moe_dispatch(idx, 6)
    assert seg.tolist() == [0, 1, 2, 2, 4, 4, 4] and perm.tolist() == [3, 1, 0, 2]
    with pytest.raises(ValueError):
        orc.moe_dispatch(np.array([[6]], np.int32), 6)


def make_experts(orc, g, E, H, I, b_in, b_mid):
    def prep(n, k, b):
        w = (g.standard_normal((E * n, k)) * 0.02).astype(np.float32)
        q, s = orc.rotate_quant_rows(w, b)
        return q.reshape(E, n, k), s.reshape(E, n)
    wg, sg = prep(I, H, b_in)
    wu, su = prep(I, H, b_in)
    wd, sd = prep(H, I, b_mid)
    return wg, sg, wu, su, wd, sd


def test_moe_ffn_equals_per_token_chain(orc):
    g = np.random.default_rng(35)
    T, H, I, E, k, b_in, b_mid = 6, 256, 256, 4, 2, 128, 256
    x = g.standard_normal((T, H)).astype(np.float32)
    wr = (g.standard_normal((E, H)) * 0.02).astype(np.float32)
    idx, w = orc.moe_route(x, wr, k)
    wg, sg, wu, su, wd, sd = make_experts(orc, g, E, H, I, b_in, b_mid)
    y, h, hq, hs, accd = orc.moe_ffn(x, idx, w, wg, sg, wu, su, wd, sd, b_in, b_mid, want_debug=True)
    perm, seg = orc.moe_dispatch(idx, E)
    qx, sx = orc.rotate_quant_rows(x, b_in)
    want = np.zeros((T, H), np.float32)
    outs = {}
    for pos, pair in enumerate(perm):
        t, e = pair // k, idx.reshape(-1)[pair]
        assert seg[e] <= pos < seg[e + 1]
        gg = orc.dequant(orc.gemm_i8_i32(qx[t:t + 1], wg[e]), sx[t:t + 1], sg[e])[0]
        uu = orc.dequant(orc.gemm_i8_i32(qx[t:t + 1], wu[e]), sx[t:t + 1], su[e])[0]
        h64 = gg.astype(np.float64) / (1 + np.exp(-gg.astype(np.float64))) * uu
        assert np.max(np.abs(h[pos] - h64)) <= 2e-6 * max(1.0, np.max(np.abs(h64)))
        hq1, hs1 = orc.rotate_quant_rows(h[pos:pos + 1], b_mid)
        assert np.array_equal(hq1[0], hq[pos]) and hs1[0] == hs[pos]
        a = orc.gemm_i8_i32(hq1, wd[e])
        assert np.array_equal(a[0], accd[pos])
        outs[pair] = orc.dequant(a, hs1, sd[e])[0]
    for t in range(T):
        acc = np.zeros(H, np.float32)
        for s in range(k):
            acc = acc + w[t, s] * outs[t * k + s]
        want[t] = acc
    assert np.array_equal(y, want)


def test_moe_ffn_h_override_and_top1_single_expert(orc):
    g = np.random.default_rng(36)
    T, H, I, E, b_in, b_mid = 3, 256, 256, 1, 128, 256
    x = g.standard_normal((T, H)).astype(np.float32)
    idx = np.zeros((T, 1), np.int32)
    w = np.ones((T, 1), np.float32)
    wg, sg, wu, su, wd, sd = make_experts(orc, g, E, H, I, b_in, b_mid)
    y, h, hq, hs, accd = orc.moe_ffn(x, idx, w, wg, sg, wu, su, wd, sd, b_in, b_mid, want_debug=True)
    # degenerate case = a plain chain of two linears around SwiGLU
    gg, _, _, _ = orc.w8a8_linear(x, wg[0], sg[0], b_in)
    uu, _, _, _ = orc.w8a8_linear(x, wu[0], su[0], b_in)
    assert np.max(np.abs(h - gg / (1 + np.exp(-gg)) * uu)) < 1e-5
    y2, _, _, _ = orc.w8a8_linear(h, wd[0], sd[0], b_mid)
    assert np.array_equal(y, y2)
    # feeding h back in reproduces everything downstream bit for bit
    y3, h3, hq3, hs3, accd3 = orc.moe_ffn(x, idx, w, wg, sg, wu, su, wd, sd, b_in, b_mid,
                                          h_in=h, want_debug=True)
    assert np.array_equal(y3, y) and np.array_equal(hq3, hq) and np.array_equal(accd3, accd)
