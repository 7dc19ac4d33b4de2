"""Pins oracle a4/a5 (int8 contraction), a6 (dequant) and a8 (GQA decode).

Integer contraction: any correct implementation is bit-exact, so brute force
and numpy int64 pin it.  Attention: float64 numpy restatement plus the special
cases that collapse to closed forms (T = 1, identical keys, shared KV head).
"""
import numpy as np
import pytest


def test_gemm_brute_force_tiny(orc):
    g = np.random.default_rng(1)
    qx = g.integers(-127, 128, (3, 17)).astype(np.int8)
    qw = g.integers(-127, 128, (5, 17)).astype(np.int8)
    want = [[sum(int(qx[m, k]) * int(qw[n, k]) for k in range(17)) for n in range(5)] for m in range(3)]
    assert orc.gemm_i8_i32(qx, qw).tolist() == want
    assert orc.gemm_i8_i32(qx, qw, scalar=True).tolist() == want


@pytest.mark.parametrize("M,N,K", [(1, 64, 4096), (16, 48, 14336), (33, 70, 1000)])
def test_gemm_vs_numpy_int64(orc, M, N, K):
    g = np.random.default_rng(M + N)
    qx = g.integers(-127, 128, (M, K)).astype(np.int8)
    qw = g.integers(-127, 128, (N, K)).astype(np.int8)
    want = qx.astype(np.int64) @ qw.astype(np.int64).T
    got = orc.gemm_i8_i32(qx, qw)
    assert np.array_equal(got.astype(np.int64), want)
    assert np.array_equal(orc.gemm_i8_i32(qx, qw, scalar=True), got)


@pytest.mark.parametrize("M,N,K", [(4, 6, 64), (5, 7, 200), (4, 6, 63), (9, 13, 128), (67, 100, 4096 + 128),
                                   (130, 50, 14336), (8, 16, 32), (3, 9, 256)])
def test_gemm_blocked_form_edges(orc, M, N, K):
    """The blocked form the oracle takes on hosts with byte dot-product instructions (register tiles of 4 x 6,
    row panels of 64, K chunks of 4096, a scalar K tail, a +128 bias on the activation codes) against the plain
    loop and numpy int64: tile and panel remainders, several K chunks, K below and off the vector width, and
    rows of -128 / -127 / 127 that push the biased partial sums to their extremes."""
    g = np.random.default_rng(M * 131 + N * 7 + K)
    qx = g.integers(-128, 128, (M, K)).astype(np.int8)
    qw = g.integers(-128, 128, (N, K)).astype(np.int8)
    qx[0, :], qw[0, :] = -128, -128
    qx[M - 1, :], qw[N - 1, :] = 127, -127
    got = orc.gemm_i8_i32(qx, qw)
    assert np.array_equal(got, orc.gemm_i8_i32(qx, qw, scalar=True))
    assert np.array_equal(got.astype(np.int64), qx.astype(np.int64) @ qw.astype(np.int64).T)


def test_gemm_extreme_values_do_not_overflow(orc):
    K = 14336
    qx = np.full((2, K), 127, np.int8)
    qx[1] = -127
    qw = np.full((2, K), 127, np.int8)
    got = orc.gemm_i8_i32(qx, qw)
    assert got[0, 0] == 127 * 127 * K and got[1, 1] == -127 * 127 * K
    assert 127 * 127 * K < 2 ** 31


def test_dequant_closed_form(orc):
    g = np.random.default_rng(2)
    acc = g.integers(-2 ** 27, 2 ** 27, (4, 6)).astype(np.int32)
    sx = g.uniform(0.01, 1, 4).astype(np.float32)
    sw = g.uniform(0.001, 0.1, 6).astype(np.float32)
    want = (acc.astype(np.float32) * sx[:, None]) * sw[None, :]
    assert np.array_equal(orc.dequant(acc, sx, sw), want)


def test_linear_is_composition_and_close_to_fp(orc):
    g = np.random.default_rng(4)
    M, K, N, b = 8, 512, 24, 128
    x = g.standard_normal((M, K)).astype(np.float32)
    w = (g.standard_normal((N, K)) * 0.02).astype(np.float32)
    qw, sw = orc.rotate_quant_rows(w, b)
    y, qx, sx, acc = orc.w8a8_linear(x, qw, sw, b)
    qx2, sx2 = orc.rotate_quant_rows(x, b)
    assert np.array_equal(qx, qx2) and np.array_equal(sx, sx2)
    assert np.array_equal(acc, orc.gemm_i8_i32(qx, qw))
    assert np.array_equal(y, orc.dequant(acc, sx, sw))
    # the rotation is orthogonal, so the quantized product approximates x @ w.T
    ref = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 0.03


def make_kv(orc, g, B, Hkv, T, D):
    k = g.standard_normal((B * Hkv * T, D)).astype(np.float32)
    v = g.standard_normal((B * Hkv * T, D)).astype(np.float32)
    kq, ks = orc.rotate_quant_rows(k, D)
    vq, vs = orc.rotate_quant_rows(v, D)
    sh = (B, Hkv, T)
    return kq.reshape(*sh, D), ks.reshape(sh), vq.reshape(*sh, D), vs.reshape(sh)


def attn_numpy_f64(orc, q, kq, ks, vq, vs):
    B, Hq, D = q.shape
    Hkv, T = kq.shape[1], kq.shape[2]
    G = Hq // Hkv
    o = np.zeros((B, Hq, D))
    qq, sq = orc.rotate_quant_rows(q.reshape(-1, D), D)
    qq, sq = qq.reshape(B, Hq, D), sq.reshape(B, Hq)
    for b in range(B):
        for h in range(Hq):
            kv = h // G
            dots = kq[b, kv].astype(np.int64) @ qq[b, h].astype(np.int64)
            s = dots * (np.float64(sq[b, h]) * ks[b, kv].astype(np.float64)) / np.sqrt(D)
            p = np.exp(s - s.max())
            p /= p.sum()
            o[b, h] = (p * vs[b, kv].astype(np.float64)) @ vq[b, kv].astype(np.float64)
    return o


def test_attention_vs_numpy_float64(orc):
    g = np.random.default_rng(21)
    B, Hq, Hkv, D, T = 2, 8, 2, 128, 77
    q = g.standard_normal((B, Hq, D)).astype(np.float32)
    kq, ks, vq, vs = make_kv(orc, g, B, Hkv, T, D)
    want_rot = attn_numpy_f64(orc, q, kq, ks, vq, vs)
    got_rot, qq, sq, dots = orc.gqa_decode(q, kq, ks, vq, vs, out_rotated=True, want_debug=True)
    assert np.max(np.abs(got_rot - want_rot)) < 1e-6
    # int32 scores against a direct integer product
    G = Hq // Hkv
    for b in range(B):
        for h in range(Hq):
            assert np.array_equal(dots[b, h].astype(np.int64),
                                  kq[b, h // G].astype(np.int64) @ qq[b, h].astype(np.int64))
    # unrotated output = one more normalized Hadamard of the rotated one
    got = orc.gqa_decode(q, kq, ks, vq, vs, out_rotated=False)
    assert np.array_equal(got.reshape(-1, D), orc.rotate_rows(got_rot.reshape(-1, D), D))


def test_attention_single_token_returns_dequantized_v(orc):
    g = np.random.default_rng(22)
    B, Hq, Hkv, D, T = 1, 4, 2, 128, 1
    q = g.standard_normal((B, Hq, D)).astype(np.float32)
    kq, ks, vq, vs = make_kv(orc, g, B, Hkv, T, D)
    o = orc.gqa_decode(q, kq, ks, vq, vs, out_rotated=True)
    for h in range(Hq):
        want = (np.float64(vs[0, h // 2, 0]) * vq[0, h // 2, 0].astype(np.float64)).astype(np.float32)
        assert np.array_equal(o[0, h], want)


def test_attention_identical_keys_average_values(orc):
    g = np.random.default_rng(23)
    B, Hq, Hkv, D, T = 1, 2, 1, 128, 33
    q = g.standard_normal((B, Hq, D)).astype(np.float32)
    kq, ks, vq, vs = make_kv(orc, g, B, Hkv, T, D)
    kq[:] = kq[:, :, :1]
    ks[:] = ks[:, :, :1]
    o = orc.gqa_decode(q, kq, ks, vq, vs, out_rotated=True)
    want = np.mean(vs[0, 0, :, None].astype(np.float64) * vq[0, 0].astype(np.float64), axis=0)
    assert np.max(np.abs(o[0, 0] - want)) < 1e-6 and np.max(np.abs(o[0, 1] - want)) < 1e-6


def test_attention_gqa_head_sharing(orc):
    g = np.random.default_rng(24)
    B, Hq, Hkv, D, T = 1, 8, 2, 128, 40
    q = g.standard_normal((B, Hq, D)).astype(np.float32)
    q[0, 1] = q[0, 0]      # same group, same query  -> same output
    q[0, 4] = q[0, 0]      # other group, same query -> generally different
    kq, ks, vq, vs = make_kv(orc, g, B, Hkv, T, D)
    o = orc.gqa_decode(q, kq, ks, vq, vs)
    assert np.array_equal(o[0, 0], o[0, 1]) and not np.array_equal(o[0, 0], o[0, 4])
    # swapping the two KV heads swaps the query groups
    o2 = orc.gqa_decode(np.concatenate([q[:, 4:], q[:, :4]], 1), kq[:, ::-1], ks[:, ::-1], vq[:, ::-1], vs[:, ::-1])
    assert np.array_equal(o2[:, :4], o[:, 4:]) and np.array_equal(o2[:, 4:], o[:, :4])


def test_attention_rejects_bad_shapes(orc):
    q = np.zeros((1, 3, 128), np.float32)
    kq = np.zeros((1, 2, 4, 128), np.int8)
    s = np.ones((1, 2, 4), np.float32)
    with pytest.raises(ValueError):
        orc.gqa_decode(q, kq, s, kq, s)
