"""Pins the oracle's decoder-layer glue (RMSNorm, rotary embedding, SwiGLU) by mathematics: float64 closed
forms, invariants and special cases chosen so that a dropped term, a wrong sign or a swapped pair fails."""
import numpy as np


def test_rmsnorm_float64_formula_and_invariants(orc):
    g = np.random.default_rng(101)
    for M, H in ((3, 64), (2, 4096), (1, 4)):
        x = g.standard_normal((M, H)).astype(np.float32) * 3
        w = (1 + 0.1 * g.standard_normal(H)).astype(np.float32)
        eps = 1e-5
        y = orc.rmsnorm(x, w, eps)
        x64 = x.astype(np.float64)
        want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + eps) * w
        assert np.max(np.abs(y - want)) <= 4e-7 * np.max(np.abs(want))
        # weight 1, eps 0: every row leaves with mean square 1; a positive row scale cancels
        y1 = orc.rmsnorm(x, np.ones(H, np.float32), 0.0)
        assert np.allclose((y1.astype(np.float64) ** 2).mean(axis=1), 1.0, atol=1e-6)
        y2 = orc.rmsnorm(x * np.float32(8.0), np.ones(H, np.float32), 0.0)   # power of two: exact in fp32
        assert np.array_equal(y1, y2)
    # eps matters where the row is small: a zero row gives zeros, not NaN
    z = orc.rmsnorm(np.zeros((1, 8), np.float32), np.ones(8, np.float32), 1e-6)
    assert not z.any()
    # a constant row c with weight g gives sign(c) * g (mean square = c^2)
    c = orc.rmsnorm(np.full((1, 16), -2.5, np.float32), np.arange(16, dtype=np.float32), 0.0)
    assert np.allclose(c[0], -np.arange(16), atol=1e-6)


def test_rmsnorm_residual_is_added_first_and_returned(orc):
    g = np.random.default_rng(102)
    x = g.standard_normal((4, 256)).astype(np.float32)
    r = g.standard_normal((4, 256)).astype(np.float32)
    w = g.standard_normal(256).astype(np.float32)
    h, y = orc.rmsnorm(x, w, 1e-5, residual=r)
    assert np.array_equal(h, x + r)                      # one fp32 add
    assert np.array_equal(y, orc.rmsnorm(x + r, w, 1e-5))


def rope_tables(T, D=128, theta=10000.0):
    inv = theta ** (-np.arange(D // 2, dtype=np.float64) * 2.0 / D)
    ang = np.arange(T, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def test_rope_is_the_complex_rotation_of_each_pair(orc):
    g = np.random.default_rng(103)
    D, T = 128, 50
    cos, sin = rope_tables(T, D)
    rows = g.standard_normal((7, D)).astype(np.float32)
    pos = np.array([0, 1, 2, 17, 49, 33, 5], np.int32)
    out = orc.rope_rows(rows, pos, cos, sin)
    z = rows[:, :64].astype(np.float64) + 1j * rows[:, 64:].astype(np.float64)
    rot = z * (cos[pos].astype(np.float64) + 1j * sin[pos].astype(np.float64))
    assert np.max(np.abs(out[:, :64] - rot.real)) <= 5e-7 and np.max(np.abs(out[:, 64:] - rot.imag)) <= 5e-7
    # position 0 (cos 1, sin 0) is the identity, exactly
    assert np.array_equal(out[0], rows[0])
    # a rotation keeps the length of every pair
    n_in = rows[:, :64].astype(np.float64) ** 2 + rows[:, 64:].astype(np.float64) ** 2
    n_out = out[:, :64].astype(np.float64) ** 2 + out[:, 64:].astype(np.float64) ** 2
    assert np.allclose(n_in, n_out, rtol=1e-6)
    # a quarter turn (cos 0, sin 1) sends (a, b) to (-b, a): the sign and the pairing are pinned
    q = orc.rope_rows(rows[:1], np.zeros(1, np.int32), np.zeros((1, 64), np.float32), np.ones((1, 64), np.float32))
    assert np.array_equal(q[0, :64], -rows[0, 64:]) and np.array_equal(q[0, 64:], rows[0, :64])


def test_rope_products_are_rounded_before_the_add(orc):
    """No fused multiply-add: the result equals the one built from fp32-rounded products."""
    g = np.random.default_rng(104)
    cos, sin = rope_tables(8)
    rows = g.standard_normal((8, 128)).astype(np.float32)
    pos = np.arange(8, dtype=np.int32)
    out = orc.rope_rows(rows, pos, cos, sin)
    a, b, c, s = rows[:, :64], rows[:, 64:], cos[pos], sin[pos]
    lo = (a * c).astype(np.float32) - (b * s).astype(np.float32)
    hi = (b * c).astype(np.float32) + (a * s).astype(np.float32)
    assert np.array_equal(out[:, :64], lo) and np.array_equal(out[:, 64:], hi)


def test_swiglu_fused_row(orc):
    g = np.random.default_rng(105)
    M, I = 5, 96
    gu = (g.standard_normal((M, 2 * I)) * 3).astype(np.float32)
    h = orc.swiglu(gu)
    g64, u64 = gu[:, :I].astype(np.float64), gu[:, I:].astype(np.float64)
    want = g64 / (1 + np.exp(-g64)) * u64
    assert np.max(np.abs(h - want)) <= 1e-6 * max(1.0, np.max(np.abs(want)))
    # gate 0 gives 0; a large gate passes g*u; a very negative gate closes
    edge = np.array([[0.0, 30.0, -30.0, 2.0, 7.0, 5.0]], np.float32)     # I = 3: gates | ups
    e = orc.swiglu(edge)
    assert e[0, 0] == 0.0 and abs(e[0, 1] - 210.0) < 1e-4 and abs(e[0, 2]) < 1e-10
