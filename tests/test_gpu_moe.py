"""GPU parity: MoE router, dispatch and grouped expert FFN.
Gates: expert indices, dispatch order, int8 codes and int32-derived outputs
bit-exact; routing weights within 2e-6; SwiGLU output (expf) within 1e-5
relative; layer output rel-L2 <= 1e-3."""
import numpy as np
import pytest

import workload

pytestmark = pytest.mark.gpu


def make_experts(orc, seed, E, H, I):
    def prep(n, k, b, stream):
        q, s = orc.rotate_quant_rows(workload.weights(seed, E * n, k, stream), b)
        return q.reshape(E, n, k), s.reshape(E, n)
    return prep(I, H, 128, 0) + prep(I, H, 128, 1) + prep(H, I, 256, 2)


def gpu_route(mi, dev, x, wr, topk):
    mark = dev.mark()
    T = x.shape[0]
    didx, dw = dev.empty((T, topk), np.int32), dev.empty((T, topk), np.float32)
    ws = dev.empty(mi.lib.mi_moe_route_workspace_bytes(T, wr.shape[0]), np.uint8)
    mi.moe_route(dev.upload(x), dev.upload(wr), didx, dw, topk, ws)
    idx, w = dev.download(didx), dev.download(dw)
    dev.reset_to(mark)
    return idx, w


@pytest.mark.parametrize("T,H,E,topk", [(512, 2048, 128, 8), (7, 256, 16, 2), (33, 512, 64, 8), (5, 1024, 256, 4),
                                        (1, 2048, 128, 1)])
def test_router_indices_exact_weights_close(mi, dev, orc, T, H, E, topk):
    x = workload.activations(41, T, H)
    wr = workload.weights(42, E, H)
    idx, w = gpu_route(mi, dev, x, wr, topk)
    idxo, wo = orc.moe_route(x, wr, topk)
    assert np.array_equal(idx, idxo)
    assert np.max(np.abs(w - wo)) <= 2e-6
    assert np.max(np.abs(w.sum(axis=1) - 1)) <= 1e-6


def test_router_ties_go_to_lower_expert(mi, dev, orc):
    x = workload.activations(43, 16, 512)
    wr = workload.weights(44, 32, 512)
    wr[9] = wr[3]
    wr[20] = wr[3]
    wr[31] = wr[30]
    idx, w = gpu_route(mi, dev, x, wr, 8)
    idxo, wo = orc.moe_route(x, wr, 8)
    assert np.array_equal(idx, idxo)
    same = np.repeat(wr[:1], 32, 0)
    idx, w = gpu_route(mi, dev, x, same, 4)
    assert np.array_equal(idx, np.tile(np.arange(4, dtype=np.int32), (16, 1)))
    assert np.allclose(w, 0.25, atol=1e-7)


@pytest.mark.parametrize("T,E,topk", [(512, 128, 8), (1, 16, 1), (37, 64, 8), (2048, 128, 8), (100, 256, 2)])
def test_dispatch_exact(mi, dev, orc, T, E, topk):
    g = np.random.default_rng(T + E)
    idx = np.stack([g.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    mark = dev.mark()
    dperm, dseg = dev.empty(T * topk, np.int32), dev.empty(E + 1, np.int32)
    mi.moe_dispatch(dev.upload(idx), dperm, dseg, E)
    perm, seg = dev.download(dperm), dev.download(dseg)
    dev.reset_to(mark)
    permo, sego = orc.moe_dispatch(idx, E)
    assert np.array_equal(seg, sego) and np.array_equal(perm, permo)


def test_dispatch_with_idle_experts(mi, dev, orc):
    T, E, topk = 64, 128, 2
    idx = np.stack([[3, 77]] * T).astype(np.int32)     # only two experts ever picked
    mark = dev.mark()
    dperm, dseg = dev.empty(T * topk, np.int32), dev.empty(E + 1, np.int32)
    mi.moe_dispatch(dev.upload(idx), dperm, dseg, E)
    perm, seg = dev.download(dperm), dev.download(dseg)
    dev.reset_to(mark)
    permo, sego = orc.moe_dispatch(idx, E)
    assert np.array_equal(seg, sego) and np.array_equal(perm, permo)


def run_ffn(mi, dev, x, idx, w, experts, layer_wr=None):
    T, H = x.shape
    wg, sg, wu, su, wd, sd = experts
    E, I, _ = wg.shape
    topk = idx.shape[1] if idx is not None else layer_wr[1]
    P = T * topk
    ws = dev.empty(mi.lib.mi_moe_ffn_workspace_bytes(T, H, I, E, topk), np.uint8)
    dy = dev.empty((T, H), np.float32)
    dev_w = [dev.upload(a) for a in experts]
    if layer_wr is None:
        mi.moe_ffn(dev.upload(x), dev.upload(idx), dev.upload(w), *dev_w, dy, ws)
    else:
        mi.moe_layer(dev.upload(x), dev.upload(layer_wr[0]), *dev_w, dy, topk, ws)
    off = lambda i: mi.lib.mi_moe_ffn_workspace_offset(i, T, H, I, E, topk)
    out = dict(
        y=dev.download(dy),
        qx=dev.download(ws.offset(off(0), (T, H), np.int8)),
        sx=dev.download(ws.offset(off(1), (T,), np.float32)),
        perm=dev.download(ws.offset(off(2), (P,), np.int32)),
        seg=dev.download(ws.offset(off(3), (E + 1,), np.int32)),
        h=dev.download(ws.offset(off(4), (P, I), np.float32)),
        hq=dev.download(ws.offset(off(5), (P, I), np.int8)),
        hs=dev.download(ws.offset(off(6), (P,), np.float32)),
        out=dev.download(ws.offset(off(7), (P, H), np.float32)),
        idx=dev.download(ws.offset(off(8), (T, topk), np.int32)),
        w=dev.download(ws.offset(off(9), (T, topk), np.float32)),
    )
    return out


def check_ffn_against_oracle(orc, x, idx, w, experts, r):
    wg, sg, wu, su, wd, sd = experts
    E, I, H = wg.shape
    topk = idx.shape[1]
    qxo, sxo = orc.rotate_quant_rows(x, 128)
    assert np.array_equal(r["qx"], qxo) and np.array_equal(r["sx"], sxo)
    permo, sego = orc.moe_dispatch(idx, E)
    assert np.array_equal(r["perm"], permo) and np.array_equal(r["seg"], sego)
    yo, ho, hqo, hso, accdo = orc.moe_ffn(x, idx, w, wg, sg, wu, su, wd, sd, 128, 256, want_debug=True)
    # SwiGLU goes through expf: tolerance gate
    assert np.max(np.abs(r["h"] - ho)) <= 1e-5 * max(1.0, float(np.max(np.abs(ho))))
    # from the GPU's own h on, everything is integer / IEEE again: bit-exact
    y2, _, hq2, hs2, accd2 = orc.moe_ffn(x, idx, w, wg, sg, wu, su, wd, sd, 128, 256, h_in=r["h"], want_debug=True)
    assert np.array_equal(r["hq"], hq2) and np.array_equal(r["hs"], hs2)
    flat = idx.reshape(-1)
    for pos in range(0, permo.size, max(1, permo.size // 97)):
        pair = permo[pos]
        want = (accd2[pos].astype(np.float32) * hs2[pos]) * sd[flat[pair]]
        assert np.array_equal(r["out"][pair], want)
    assert np.array_equal(r["y"], y2)
    rel = np.linalg.norm(r["y"].astype(np.float64) - yo) / np.linalg.norm(yo.astype(np.float64))
    assert rel <= 1e-3
    return rel


@pytest.mark.parametrize("T,H,I,E,topk", [(24, 256, 256, 16, 2), (70, 512, 768, 64, 8), (9, 2048, 256, 16, 1),
                                          # hidden and inner sizes past what a wave keeps in registers: the kernels that stream
                                          # the activation rows through the ring as well
                                          (6, 4352, 1280, 16, 2)])
def test_ffn_stagewise(mi, dev, orc, T, H, I, E, topk):
    mark = dev.mark()
    x = workload.activations(51, T, H)
    wr = workload.weights(52, E, H)
    idx, w = orc.moe_route(x, wr, topk)
    experts = make_experts(orc, 53, E, H, I)
    r = run_ffn(mi, dev, x, idx, w, experts)
    check_ffn_against_oracle(orc, x, idx, w, experts, r)
    dev.reset_to(mark)


def test_ffn_skewed_routing_many_rows_per_expert(mi, dev, orc):
    """All tokens pick the same two experts: segments of 100 rows (several
    32-row passes) and 14 idle experts."""
    mark = dev.mark()
    T, H, I, E, topk = 100, 256, 256, 16, 2
    x = workload.activations(54, T, H)
    idx = np.tile(np.array([[11, 2]], np.int32), (T, 1))
    w = np.tile(np.array([[0.7, 0.3]], np.float32), (T, 1))
    experts = make_experts(orc, 55, E, H, I)
    r = run_ffn(mi, dev, x, idx, w, experts)
    check_ffn_against_oracle(orc, x, idx, w, experts, r)
    dev.reset_to(mark)


def test_ffn_slot_with_an_expert_out_of_range_contributes_nothing(mi, dev, orc):
    """A caller-made idx with an index outside [0, E): that pair is never dispatched, its row of the workspace is
    never written, and the combine leaves it out: y equals the FFN over the remaining slots."""
    mark = dev.mark()
    T, H, I, E, topk = 12, 256, 256, 16, 2
    x = workload.activations(56, T, H)
    g = np.random.default_rng(56)
    idx = np.stack([g.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    w = g.random((T, topk)).astype(np.float32)
    experts = make_experts(orc, 57, E, H, I)
    bad = idx.copy()
    bad[3, 1], bad[7, 0] = E + 5, -1
    # poison the workspace so that a stale row would show
    ws_bytes = mi.lib.mi_moe_ffn_workspace_bytes(T, H, I, E, topk)
    junk = dev.empty(ws_bytes, np.uint8)
    mi.check(mi.lib.mi_fill_u32(junk.ptr, 0x7fc00000, ws_bytes // 4, None))
    dev.sync()
    dev.reset_to(mark)
    r = run_ffn(mi, dev, x, bad, w, experts)
    # the same with weight 0 on those slots and a valid (unused) expert in their place
    ok_idx, w0 = idx.copy(), w.copy()
    w0[3, 1] = w0[7, 0] = 0.0
    for t, s_ in ((3, 1), (7, 0)):
        ok_idx[t, s_] = next(e for e in range(E) if e not in ok_idx[t])
    yo = orc.moe_ffn(x, ok_idx, w0, *experts, 128, 256)
    assert np.all(np.isfinite(r["y"]))
    assert np.linalg.norm(r["y"] - yo) <= 1e-3 * np.linalg.norm(yo)
    dev.reset_to(mark)


def test_full_layer_cfg4(mi, dev, orc):
    """512 tokens, hidden 2048, 128 experts, top-8, inner 768."""
    mark = dev.mark()
    c = workload.MOE
    T, H, E, topk, I = c["T"], c["H"], c["E"], c["topk"], c["I"]
    x = workload.activations(61, T, H)
    wr = workload.weights(62, E, H)
    experts = make_experts(orc, 63, E, H, I)
    r = run_ffn(mi, dev, x, None, None, experts, layer_wr=(wr, topk))
    idxo, wo = orc.moe_route(x, wr, topk)
    assert np.array_equal(r["idx"], idxo)
    assert np.max(np.abs(r["w"] - wo)) <= 2e-6
    # the FFN is then held to the oracle run on the GPU's own routing weights
    rel = check_ffn_against_oracle(orc, x, r["idx"], r["w"], experts, r)
    yo = orc.moe_ffn(x, idxo, wo, *experts, 128, 256)
    rel2 = np.linalg.norm(r["y"].astype(np.float64) - yo) / np.linalg.norm(yo.astype(np.float64))
    assert rel2 <= 1e-3
    assert r["seg"][E] == T * topk
    dev.reset_to(mark)


def test_argument_errors(mi, dev):
    lib = mi.lib
    mark = dev.mark()
    b = dev.empty(1 << 16, np.uint8)
    rargs = (b.ptr, b.ptr, b.ptr, b.ptr)
    assert lib.mi_moe_route(*rargs, 4, 100, 16, 2, b.ptr, b.nbytes, None) == mi.EINVAL    # H % 256
    assert lib.mi_moe_route(*rargs, 4, 256, 24, 2, b.ptr, b.nbytes, None) == mi.EINVAL    # E % 16
    assert lib.mi_moe_route(*rargs, 4, 256, 16, 9, b.ptr, b.nbytes, None) == mi.EINVAL    # topk > 8
    assert lib.mi_moe_route(*rargs, 4, 256, 512, 2, b.ptr, b.nbytes, None) == mi.ERANGE   # E > 256
    assert lib.mi_moe_route(*rargs, 4, 256, 16, 2, b.ptr, 16, None) == mi.ENOSPC          # logits do not fit
    assert lib.mi_moe_dispatch(b.ptr, b.ptr, b.ptr, 1 << 20, 128, 8, None) == mi.ERANGE      # bitmap too large
    assert lib.mi_moe_ffn_workspace_bytes(8, 200, 256, 16, 2) == mi.EINVAL                   # H % 128
    assert lib.mi_moe_ffn_workspace_bytes(8, 256, 300, 16, 2) == mi.EINVAL                   # I % 256
    args = (b.ptr,) * 10
    assert lib.mi_moe_ffn(*args, 8, 256, 256, 16, 2, b.ptr, 64, None) == mi.ENOSPC
    dev.reset_to(mark)
