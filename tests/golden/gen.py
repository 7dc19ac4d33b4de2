"""Deterministic inputs for the golden fixtures: integer hashing only (splitmix64), so the arrays do not depend on
any random-number library or its version.  Shared by make_fixtures.py (which writes the expected outputs) and by
tests/test_golden.py (which rebuilds the inputs and compares)."""
import numpy as np

_M = np.uint64(0xFFFFFFFFFFFFFFFF)


def bits(n, salt):
    """n 64-bit words of splitmix64 started at salt * golden ratio."""
    with np.errstate(over="ignore"):
        z = (np.arange(1, n + 1, dtype=np.uint64) + np.uint64(salt)) * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def bell(shape, salt, scale=1.0):
    """fp32 values with a bell-shaped distribution (sum of four 16-bit uniforms, centred), standard deviation
    about `scale`; every value is an integer times a power of two times scale, so it is exact in fp32."""
    n = int(np.prod(shape))
    z = bits(n, salt)
    s = np.zeros(n, np.int64)
    for k in range(4):
        s += ((z >> np.uint64(16 * k)) & np.uint64(0xFFFF)).astype(np.int64)
    v = (s - 2 * 65535).astype(np.float32) * np.float32(1.0 / 37837.0)   # sigma of the sum is 37837
    return (v * np.float32(scale)).reshape(shape)


def codes(shape, salt):
    """int8 codes in [-127, 127]."""
    n = int(np.prod(shape))
    return ((bits(n, salt) >> np.uint64(40)) % np.uint64(255)).astype(np.int64).astype(np.int16).__sub__(127) \
        .astype(np.int8).reshape(shape)


def scales(n, salt, lo, hi):
    u = (bits(n, salt) >> np.uint64(40)).astype(np.float64) / float(1 << 24)
    return (lo + (hi - lo) * u).astype(np.float32)


# the cases: small enough for the oracle to finish at once, shaped to touch every DECISION
FWHT = [("b128", (5, 384), 128, 11), ("b256", (3, 768), 256, 12), ("head", (6, 128), 128, 13)]
GEMM = (7, 32, 256, 21)                     # M, N, K, salt
LINEAR = (4, 32, 256, 128, 31)              # M, N, K, block, salt
ATTN = (2, 8, 2, 37, 41)                    # B, Hq, Hkv, T, salt
MOE = (6, 256, 256, 16, 4, 51)              # T, H, I, E, topk, salt
LAYER = (3, 256, 1e-5, 61)                  # rows, width, eps, salt
ROPE = (4, 10, 71)                          # rows, table positions, salt


def fwht_input(shape, salt):
    x = bell(shape, salt)
    x[0, :] = 0.0                           # all-zero row: scale 1, codes 0
    x[1, 5] *= 40.0                         # an outlier channel
    return x


def moe_inputs():
    T, H, I, E, topk, salt = MOE
    x = bell((T, H), salt)
    wr = bell((E, H), salt + 1, 0.05)
    wg, wu, wd = codes((E, I, H), salt + 2), codes((E, I, H), salt + 3), codes((E, H, I), salt + 4)
    sg, su, sd = scales(E * I, salt + 5, 1e-3, 3e-3).reshape(E, I), scales(E * I, salt + 6, 1e-3, 3e-3).reshape(E, I), \
        scales(E * H, salt + 7, 1e-3, 3e-3).reshape(E, H)
    return x, wr, wg, sg, wu, su, wd, sd


def attn_inputs():
    B, Hq, Hkv, T, salt = ATTN
    q = bell((B, Hq, 128), salt)
    kq, vq = codes((B, Hkv, T, 128), salt + 1), codes((B, Hkv, T, 128), salt + 2)
    ks = scales(B * Hkv * T, salt + 3, 5e-3, 3e-2).reshape(B, Hkv, T)
    vs = scales(B * Hkv * T, salt + 4, 5e-3, 3e-2).reshape(B, Hkv, T)
    return q, kq, ks, vq, vs


def rope_tables(npos, salt):
    """cos / sin tables [npos, 64] in fp32 (any values are legal tables: the operator only multiplies and adds)."""
    ang = (np.arange(npos, dtype=np.float64)[:, None] * (10000.0 ** (-np.arange(64, dtype=np.float64) / 64.0))[None, :])
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
