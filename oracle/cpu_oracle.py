"""ctypes front end of the CPU oracle (oracle/oracle.c).  TEST INFRASTRUCTURE.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import
this module, and only as the checker.  The arithmetic and every DECISION it
fixes are documented at the top of oracle.c; the upstream repository holds no
implementation of this path (its README.md:4, README.md:10-13), so nothing
here mirrors an upstream function.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_router_dot.restype = C.c_float
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


i64 = C.c_int64


def fwht_block(x):
    x = _c(x, np.float32).copy()
    lib().orc_fwht_block(_p(x), C.c_int(x.size))
    return x


def rotate_rows(x, b):
    x = _c(x, np.float32)
    M, K = x.shape
    out = np.empty_like(x)
    rc = lib().orc_rotate_rows(_p(x), i64(M), i64(K), C.c_int(b), _p(out))
    if rc:
        raise ValueError("orc_rotate_rows rc=%d" % rc)
    return out


def quant_row(xr):
    xr = _c(xr, np.float32)
    q = np.empty(xr.shape, np.int8)
    s = np.empty(1, np.float32)
    lib().orc_quant_row(_p(xr), i64(xr.size), _p(q), _p(s))
    return q, s[0]


def rotate_quant_rows(x, b, want_rot=False):
    x = _c(x, np.float32)
    M, K = x.shape
    q = np.empty((M, K), np.int8)
    s = np.empty(M, np.float32)
    xr = np.empty((M, K), np.float32) if want_rot else None
    rc = lib().orc_rotate_quant_rows(_p(x), i64(M), i64(K), C.c_int(b), _p(q), _p(s), _p(xr))
    if rc:
        raise ValueError("orc_rotate_quant_rows rc=%d" % rc)
    return (q, s, xr) if want_rot else (q, s)


def gemm_i8_i32(qx, qw, scalar=False):
    qx = _c(qx, np.int8)
    qw = _c(qw, np.int8)
    M, K = qx.shape
    N, K2 = qw.shape
    assert K == K2
    acc = np.empty((M, N), np.int32)
    fn = lib().orc_gemm_i8_i32_scalar if scalar else lib().orc_gemm_i8_i32
    fn(_p(qx), _p(qw), _p(acc), i64(M), i64(N), i64(K))
    return acc


def dequant(acc, sx, sw):
    acc = _c(acc, np.int32)
    sx = _c(sx, np.float32)
    sw = _c(sw, np.float32)
    M, N = acc.shape
    y = np.empty((M, N), np.float32)
    lib().orc_dequant(_p(acc), _p(sx), _p(sw), _p(y), i64(M), i64(N))
    return y


def w8a8_linear(x, qw, sw, b):
    """returns y, qx, sx, acc"""
    x = _c(x, np.float32)
    qw = _c(qw, np.int8)
    sw = _c(sw, np.float32)
    M, K = x.shape
    N = qw.shape[0]
    y = np.empty((M, N), np.float32)
    qx = np.empty((M, K), np.int8)
    sx = np.empty(M, np.float32)
    acc = np.empty((M, N), np.int32)
    rc = lib().orc_w8a8_linear(_p(x), _p(qw), _p(sw), _p(y), i64(M), i64(N), i64(K),
                               C.c_int(b), _p(qx), _p(sx), _p(acc))
    if rc:
        raise ValueError("orc_w8a8_linear rc=%d" % rc)
    return y, qx, sx, acc


def gqa_decode(q, kq, ks, vq, vs, out_rotated=False, want_debug=False):
    q = _c(q, np.float32)
    kq = _c(kq, np.int8)
    vq = _c(vq, np.int8)
    ks = _c(ks, np.float32)
    vs = _c(vs, np.float32)
    B, Hq, D = q.shape
    _, Hkv, T, _ = kq.shape
    o = np.empty((B, Hq, D), np.float32)
    qq = np.empty((B, Hq, D), np.int8) if want_debug else None
    sq = np.empty((B, Hq), np.float32) if want_debug else None
    dots = np.empty((B, Hq, T), np.int32) if want_debug else None
    rc = lib().orc_gqa_decode(_p(q), _p(kq), _p(ks), _p(vq), _p(vs), _p(o), i64(B), i64(Hq),
                              i64(Hkv), i64(D), i64(T), C.c_int(1 if out_rotated else 0),
                              _p(qq), _p(sq), _p(dots))
    if rc:
        raise ValueError("orc_gqa_decode rc=%d" % rc)
    return (o, qq, sq, dots) if want_debug else o


def router_dot(x, w):
    x = _c(x, np.float32)
    w = _c(w, np.float32)
    return np.float32(lib().orc_router_dot(_p(x), _p(w), i64(x.size)))


def moe_route(x, wr, topk, want_logits=False):
    x = _c(x, np.float32)
    wr = _c(wr, np.float32)
    T, H = x.shape
    E = wr.shape[0]
    idx = np.empty((T, topk), np.int32)
    w = np.empty((T, topk), np.float32)
    lg = np.empty((T, E), np.float32) if want_logits else None
    rc = lib().orc_moe_route(_p(x), _p(wr), i64(T), i64(H), i64(E), C.c_int(topk),
                             _p(idx), _p(w), _p(lg))
    if rc:
        raise ValueError("orc_moe_route rc=%d" % rc)
    return (idx, w, lg) if want_logits else (idx, w)


def moe_dispatch(idx, E):
    idx = _c(idx, np.int32).reshape(-1)
    perm = np.empty(idx.size, np.int32)
    seg = np.empty(E + 1, np.int32)
    rc = lib().orc_moe_dispatch(_p(idx), i64(idx.size), i64(E), _p(perm), _p(seg))
    if rc:
        raise ValueError("orc_moe_dispatch rc=%d" % rc)
    return perm, seg


def moe_ffn(x, idx, w, wg, sg, wu, su, wd, sd, b_in, b_mid, h_in=None, want_debug=False):
    """y, or (y, h, hq, hs, accd) in sorted-pair order when want_debug."""
    x = _c(x, np.float32)
    idx = _c(idx, np.int32)
    w = _c(w, np.float32)
    wg, wu, wd = _c(wg, np.int8), _c(wu, np.int8), _c(wd, np.int8)
    sg, su, sd = _c(sg, np.float32), _c(su, np.float32), _c(sd, np.float32)
    T, H = x.shape
    E, I, _ = wg.shape
    topk = idx.shape[1]
    P = T * topk
    y = np.empty((T, H), np.float32)
    if h_in is not None:
        h_in = _c(h_in, np.float32)
    h = np.empty((P, I), np.float32) if want_debug else None
    hq = np.empty((P, I), np.int8) if want_debug else None
    hs = np.empty(P, np.float32) if want_debug else None
    accd = np.empty((P, H), np.int32) if want_debug else None
    rc = lib().orc_moe_ffn(_p(x), _p(idx), _p(w), _p(wg), _p(sg), _p(wu), _p(su), _p(wd), _p(sd),
                           _p(y), i64(T), i64(H), i64(I), i64(E), C.c_int(topk), C.c_int(b_in),
                           C.c_int(b_mid), _p(h_in), _p(h), _p(hq), _p(hs), _p(accd))
    if rc:
        raise ValueError("orc_moe_ffn rc=%d" % rc)
    return (y, h, hq, hs, accd) if want_debug else y


def rmsnorm(x, g, eps, residual=None):
    """D10.  Returns y, or (h, y) when a residual is added first."""
    x = _c(x, np.float32)
    M, H = x.shape
    g = _c(g, np.float32)
    y = np.empty((M, H), np.float32)
    res = _c(residual, np.float32) if residual is not None else None
    h = np.empty((M, H), np.float32) if residual is not None else None
    rc = lib().orc_rmsnorm(_p(x), _p(res), _p(g), C.c_float(eps), _p(h), _p(y), i64(M), i64(H))
    if rc:
        raise ValueError("orc_rmsnorm rc=%d" % rc)
    return (h, y) if residual is not None else y


def rope_rows(rows, pos, cos, sin):
    """D11 on fp32 [R, D] rows (a copy is returned); row r takes table row pos[r]."""
    rows = np.array(rows, np.float32, order="C", copy=True)
    R, D = rows.shape
    pos = _c(pos, np.int32)
    rc = lib().orc_rope_rows(_p(rows), _p(pos), _p(_c(cos, np.float32)), _p(_c(sin, np.float32)), i64(R), i64(D))
    if rc:
        raise ValueError("orc_rope_rows rc=%d" % rc)
    return rows


def swiglu(gate_up):
    """D12: fp32 [M, 2I] -> [M, I]."""
    gu = _c(gate_up, np.float32)
    M, I2 = gu.shape
    h = np.empty((M, I2 // 2), np.float32)
    rc = lib().orc_swiglu(_p(gu), _p(h), i64(M), i64(I2 // 2))
    if rc:
        raise ValueError("orc_swiglu rc=%d" % rc)
    return h


def num_threads():
    return int(lib().orc_num_threads())


def pin_threads(cpus):
    """thread t of the OpenMP team -> cpus[t]; returns how many threads were pinned"""
    a = np.ascontiguousarray(cpus, dtype=np.int32)
    return int(lib().orc_pin_threads(_p(a), C.c_int(a.size)))
