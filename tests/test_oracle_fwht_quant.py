"""Pins oracle a1 (block Hadamard) and a2/a3 (row quantizer) by mathematics.

The upstream repository has no vectors for this path, so each check is chosen
so that a plausible slip (wrong stage pairing, dropped scale, truncation
instead of round-half-even, scale from the wrong row) fails one of them.
"""
import numpy as np
import pytest
import scipy.linalg


def sylvester(b):
    h = np.array([[1.0]])
    while h.shape[0] < b:
        h = np.block([[h, h], [h, -h]])
    return h


@pytest.mark.parametrize("b", [2, 4, 8, 128, 256])
def test_sylvester_matches_scipy(b):
    assert np.array_equal(sylvester(b), scipy.linalg.hadamard(b).astype(np.float64))


@pytest.mark.parametrize("b", [2, 8, 128, 256])
def test_fwht_equals_explicit_matrix(orc, b):
    g = np.random.default_rng(b)
    x = g.standard_normal(b).astype(np.float32)
    want = sylvester(b) @ x.astype(np.float64) / np.sqrt(b)
    got = orc.fwht_block(x)
    assert np.max(np.abs(got - want)) <= 4e-6 * np.linalg.norm(want)


@pytest.mark.parametrize("b", [128, 256])
def test_fwht_unit_vectors_give_signed_columns(orc, b):
    s = np.float32(1.0 / np.sqrt(b))
    for j in (0, 1, 5, b // 2, b - 1):
        e = np.zeros(b, np.float32)
        e[j] = 1.0
        got = orc.fwht_block(e)
        sign = np.array([(-1) ** bin(i & j).count("1") for i in range(b)], np.float32)
        assert np.array_equal(got, sign * s)


def test_fwht_integer_inputs_exact(orc):
    g = np.random.default_rng(7)
    for b in (128, 256):
        x = g.integers(-1000, 1000, b).astype(np.float32)
        hx = (sylvester(b) @ x.astype(np.float64))
        want = hx.astype(np.float32) * np.float32(1.0 / np.sqrt(b))  # one rounding
        assert np.array_equal(orc.fwht_block(x), want)
    # b = 256: the scale is exactly 1/16
    assert np.float32(1.0 / np.sqrt(256)) == np.float32(0.0625)


@pytest.mark.parametrize("b", [128, 256])
def test_fwht_involution_and_norm(orc, b):
    g = np.random.default_rng(3)
    x = g.standard_normal(b).astype(np.float32)
    y = orc.fwht_block(x)
    assert abs(np.linalg.norm(y.astype(np.float64)) / np.linalg.norm(x.astype(np.float64)) - 1) < 1e-6
    z = orc.fwht_block(y)
    assert np.max(np.abs(z - x)) < 2e-6 * np.max(np.abs(x)) * np.log2(b)


def fwht_numpy_f32(x, b):
    """Independent fp32 restatement of the stage order: reshape-based."""
    x = x.astype(np.float32).copy()
    h = 1
    while h < b:
        v = x.reshape(-1, b // (2 * h), 2, h)
        u, w = v[:, :, 0, :].copy(), v[:, :, 1, :].copy()
        v[:, :, 0, :] = u + w
        v[:, :, 1, :] = u - w
        h *= 2
    return x * np.float32(1.0 / np.sqrt(b))


@pytest.mark.parametrize("b,K", [(128, 4096), (256, 768), (128, 128)])
def test_rotate_rows_bit_exact_vs_numpy_fp32(orc, b, K):
    g = np.random.default_rng(11)
    x = g.standard_normal((5, K)).astype(np.float32)
    want = fwht_numpy_f32(x.reshape(-1, b), b).reshape(5, K)
    assert np.array_equal(orc.rotate_rows(x, b), want)


def test_rotate_rejects_bad_block(orc):
    x = np.zeros((1, 96), np.float32)
    with pytest.raises(ValueError):
        orc.rotate_rows(x, 128)
    with pytest.raises(ValueError):
        orc.rotate_rows(x, 96)


def test_quant_round_half_even_and_clamp(orc):
    # a = 127 makes inv == 1 and scale == 1 exactly, so codes are rintf(x)
    x = np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5, 3.49, -3.51, 0.0], np.float32)
    q, s = orc.quant_row(x)
    assert s == np.float32(1.0)
    assert q.tolist() == [127, 0, 2, 2, 0, -2, -2, 126, -126, 3, -4, 0]


def test_quant_zero_row(orc):
    q, s = orc.quant_row(np.zeros(256, np.float32))
    assert s == np.float32(1.0) and not q.any()


def test_quant_invariants(orc):
    g = np.random.default_rng(5)
    x = (g.standard_normal((64, 512)) * g.uniform(1e-3, 1e3, (64, 1))).astype(np.float32)
    for r in x:
        q, s = orc.quant_row(r)
        assert np.max(np.abs(q.astype(np.int32))) == 127
        assert s == np.float32(np.max(np.abs(r))) / np.float32(127.0)
        err = np.abs(r.astype(np.float64) - q.astype(np.float64) * np.float64(s))
        assert np.max(err) <= 0.5 * np.float64(s) * (1 + 1e-5)
        qn, sn = orc.quant_row(-r)
        assert sn == s and np.array_equal(qn, -q)


def test_quant_bit_exact_vs_numpy_fp32(orc):
    g = np.random.default_rng(9)
    x = g.standard_normal((16, 1024)).astype(np.float32)
    for r in x:
        a = np.max(np.abs(r))
        inv = np.float32(127.0) / a
        want = np.clip(np.rint(r * inv), -127, 127).astype(np.int8)
        q, s = orc.quant_row(r)
        assert np.array_equal(q, want) and s == a / np.float32(127.0)


def test_rotate_quant_rows_is_composition(orc):
    g = np.random.default_rng(13)
    x = g.standard_normal((7, 768)).astype(np.float32)
    q, s, xr = orc.rotate_quant_rows(x, 256, want_rot=True)
    assert np.array_equal(xr, orc.rotate_rows(x, 256))
    for m in range(7):
        qm, sm = orc.quant_row(xr[m])
        assert np.array_equal(q[m], qm) and s[m] == sm
    # scale belongs to its own row: scaling one row must not move another
    x2 = x.copy()
    x2[3] *= 8
    q2, s2 = orc.rotate_quant_rows(x2, 256)
    assert np.array_equal(np.delete(q2, 3, 0), np.delete(q, 3, 0))
    assert s2[3] == s[3] * 8 and np.array_equal(q2[3], q[3])


def test_quant_non_finite_values_are_defined(orc):
    """D14: a NaN takes no part in the absmax and gets -127; +-Inf makes the scale Inf, finite values 0 and the
    infinite ones -127; NaNs among zeros only: scale 1."""
    row = np.array([1.0, -2.0, np.nan, 0.5], np.float32)
    q, s = orc.quant_row(row)
    assert s == np.float32(2.0) / np.float32(127.0) and list(q) == [64, -127, -127, 32]
    row = np.array([1.0, np.inf, -np.inf, -3.0, 0.0], np.float32)
    q, s = orc.quant_row(row)
    assert np.isinf(s) and s > 0 and list(q) == [0, -127, -127, 0, 0]
    row = np.array([0.0, np.nan, -0.0], np.float32)
    q, s = orc.quant_row(row)
    assert s == 1.0 and list(q) == [0, -127, 0]
