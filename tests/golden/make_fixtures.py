"""Writes tests/golden/hotpath.npz: expected outputs of the CPU oracle (oracle/oracle.c) on the small deterministic
cases of gen.py.  There is no upstream code or vector for this path, so these are the oracle's own outputs, taken
after tests/test_oracle_*.py had pinned it by mathematics; they freeze its DECISIONS as data: a later change of
rounding, order or tie-break in the oracle or in a kernel shows up as a difference from this file.

    python tests/golden/make_fixtures.py        (rewrites the file; commit it)
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
sys.path.insert(0, os.path.join(HERE, "..", "..", "oracle"))
import cpu_oracle as orc   # noqa: E402
import gen                 # noqa: E402


def main():
    out = {}
    for name, shape, block, salt in gen.FWHT:
        x = gen.fwht_input(shape, salt)
        q, s, xr = orc.rotate_quant_rows(x, block, want_rot=True)
        out["fwht_%s_q" % name], out["fwht_%s_s" % name], out["fwht_%s_rot" % name] = q, s, xr
    M, N, K, salt = gen.GEMM
    out["gemm_acc"] = orc.gemm_i8_i32(gen.codes((M, K), salt), gen.codes((N, K), salt + 1))
    M, N, K, b, salt = gen.LINEAR
    qw, sw = orc.rotate_quant_rows(gen.bell((N, K), salt + 1, 0.02), b)
    y, qx, sx, acc = orc.w8a8_linear(gen.fwht_input((M, K), salt), qw, sw, b)
    out["linear_qw"], out["linear_sw"], out["linear_y"], out["linear_acc"] = qw, sw, y, acc
    q, kq, ks, vq, vs = gen.attn_inputs()
    o, qq, sq, dots = orc.gqa_decode(q, kq, ks, vq, vs, out_rotated=False, want_debug=True)
    out["attn_o"], out["attn_qq"], out["attn_sq"], out["attn_dots"] = o, qq, sq, dots
    out["attn_o_rot"] = orc.gqa_decode(q, kq, ks, vq, vs, out_rotated=True)
    T, H, I, E, topk, salt = gen.MOE
    x, wr, wg, sg, wu, su, wd, sd = gen.moe_inputs()
    idx, w, lg = orc.moe_route(x, wr, topk, want_logits=True)
    perm, seg = orc.moe_dispatch(idx, E)
    yy, h, hq, hs, accd = orc.moe_ffn(x, idx, w, wg, sg, wu, su, wd, sd, 128, 256, want_debug=True)
    out.update(moe_idx=idx, moe_w=w, moe_logits=lg, moe_perm=perm, moe_seg=seg, moe_y=yy, moe_h=h, moe_hq=hq,
               moe_hs=hs)
    R, W, eps, salt = gen.LAYER
    xx, res, g = gen.bell((R, W), salt), gen.bell((R, W), salt + 1), gen.bell((W,), salt + 2, 0.3) + np.float32(1)
    out["rms_h"], out["rms_y"] = orc.rmsnorm(xx, g, eps, residual=res)
    out["swiglu_h"] = orc.swiglu(gen.bell((R, 2 * W), salt + 3, 2.0))
    rows, npos, salt = gen.ROPE
    cos, sin = gen.rope_tables(npos, salt)
    pos = np.array([0, 3, 9, 3], np.int32)[:rows]
    out["rope_cos"], out["rope_sin"], out["rope_pos"] = cos, sin, pos
    src = gen.bell((rows, 128), salt)
    out["rope_out"] = orc.rope_rows(src, pos, cos, sin)
    # the cache append of a decode step: the key head is rotated (rotary, then Hadamard) and quantized, the value head
    # only Hadamard-rotated and quantized
    out["rope_kq"], out["rope_ks"] = orc.rotate_quant_rows(out["rope_out"], 128)
    out["rope_vq"], out["rope_vs"] = orc.rotate_quant_rows(src, 128)
    path = os.path.join(HERE, "hotpath.npz")
    np.savez_compressed(path, **out)
    print("wrote %s: %d arrays, %d bytes" % (path, len(out), os.path.getsize(path)))


if __name__ == "__main__":
    main()
