"""The work list of the batched GEMM, checked on the host (no device call): every output element of every problem
is covered by a tile that lies inside its matrix, every address the kernel forms from a tile stays inside the
operands and inside the kernel's LDS areas, and the list is balanced."""
import ctypes as C

import numpy as np
import pytest

BM, BN = 256, 256
CFG3 = [(2048, 6144, 4096), (2048, 14336, 4096), (2048, 14336, 4096), (2048, 4096, 14336)]


def plan(mi, shapes, cus=256):
    n = len(shapes)
    mnk = (C.c_int64 * (3 * n))(*[v for s in shapes for v in s])
    cap = 64 << 20
    buf = np.empty(cap // 4, np.int32)
    per_wg = C.c_int32()
    nbytes = mi.lib.mi_gemm_batch_plan_host(mnk, n, cus, buf.ctypes.data, cap, C.byref(per_wg))
    assert nbytes > 0, nbytes
    assert nbytes == cus * per_wg.value * 16
    return buf[:nbytes // 4].reshape(cus, per_wg.value, 4)


@pytest.mark.parametrize("shapes,cus", [
    (CFG3, 256), ([(300, 272, 512)], 256), ([(256, 256, 384)], 256), ([(2048, 6144, 384)] * 8, 256),
    ([(1000, 1008, 384), (4096, 272, 512)], 64), (CFG3, 304), ([(777, 4096, 1024)], 7),
])
def test_every_output_is_covered_once_or_with_equal_tiles(mi, shapes, cus):
    lists = plan(mi, shapes, cus)
    cover = [np.zeros((M, N), np.uint8) for M, N, K in shapes]
    for w in range(cus):
        ended = False
        for p, m0, n0, cost in lists[w]:
            if p < 0:
                ended = True
                continue
            assert not ended, "an entry behind the end mark"
            M, N, K = shapes[p]
            assert 0 <= m0 <= M - BM and 0 <= n0 <= N - BN and n0 % 16 == 0
            assert cost == K // 128 + 10
            cover[p][m0:m0 + BM, n0:n0 + BN] += 1
        assert ended, "every list ends with a mark"
    for c, (M, N, K) in zip(cover, shapes):
        assert c.min() >= 1
        # only the last row / column of tiles is moved inwards: at most four tiles meet in a corner
        assert c.max() <= 4
        tiles = -(-M // BM) * -(-N // BN)
        assert int(c.sum()) == tiles * BM * BN


def test_addresses_formed_from_a_tile_stay_inside(mi):
    """Replays the kernel's address arithmetic for the first and last tile rows/columns of a problem: global byte
    offsets of the direct-to-LDS loads (wave w of eight fills blocks w + 8q: row (w + 8q) * 8 + rho of the tile,
    chunk c ^ sigma of a 128-byte K stage; the offset is formed in 32 bits), their LDS targets (two activation and three
    weight stage buffers fill the unit's 160 KB) and the loads of a lane's scales."""
    NBX, NBW = BM // 8, BN // 8          # 1 KB blocks (8 rows x 128 B) per stage
    XSTAGE, WSTAGE = NBX * 1024, NBW * 1024
    XAREA, STAGES = 2 * XSTAGE, 2 * XSTAGE + 3 * WSTAGE
    assert STAGES == 160 * 1024
    for M, N, K in [(2048, 14336, 4096), (300, 272, 512), (256, 256, 384), (2048, 4096, 14336)]:
        lists = plan(mi, [(M, N, K)])
        tiles = lists[lists[:, :, 0] >= 0]
        for _, m0, n0, _ in tiles[[0, -1]]:
            for w in range(8):
                for lane in range(64):
                    rho, c = lane >> 3, lane & 7
                    sigma = ((w & 1) << 2) | (rho >> 1)
                    voff = (w * 8 + rho) * K + ((c ^ sigma) << 4)
                    for kt in (0, K // 128 - 1):
                        for rows, base, nq, lds0, stage, nbuf, lo, hi in (
                                (M, m0, NBX // 8, w * 1024, XSTAGE, 2, 0, XAREA),
                                (N, n0, NBW // 8, XAREA + w * 1024, WSTAGE, 3, XAREA, STAGES)):
                            for q in range(nq):
                                off32 = voff + kt * 128 + q * 64 * K      # what the lane adds to the tile's base
                                assert 0 <= off32 < 1 << 32
                                off = base * K + off32
                                assert 0 <= off and off + 16 <= rows * K
                                for buf in range(nbuf):
                                    lds = lds0 + buf * stage + q * 8192 + 16 * lane
                                    assert lo <= lds and lds + 16 <= hi
            # a lane's scales: wave (wm, wn), lane (r, g): rows m0 + 64 wm + 16 i + r % 8 (+ 8), four columns from
            # n0 + 128 wn + 32 jp + (16 if r >= 8) + 4 g
            for w in range(8):
                wm, wn = w >> 1, w & 1
                for lane in range(64):
                    r, g = lane & 15, lane >> 4
                    for i in range(4):
                        for half in (0, 8):
                            assert 0 <= m0 + 64 * wm + 16 * i + half + (r & 7) < M
                    for jp in range(4):
                        c0 = n0 + 128 * wn + 32 * jp + (16 if r >= 8 else 0) + 4 * g
                        assert 0 <= c0 and c0 + 4 <= N


def test_cfg3_list_is_balanced(mi):
    lists = plan(mi, CFG3)
    load = np.where(lists[:, :, 0] >= 0, lists[:, :, 3], 0).sum(axis=1)
    assert load.min() > 0
    # 1,216 tiles in rounds of 256: the longest list exceeds the mean by less than a tenth
    assert load.max() <= load.mean() * 1.10, (load.max(), load.mean())
    # workgroup id mod 8 is the XCD: the XCDs' totals differ by at most one short tile per workgroup
    per_xcd = np.array([load[x::8].max() for x in range(8)])
    assert per_xcd.max() - per_xcd.min() <= 4096 // 128 + 10, per_xcd
    # all workgroups of an XCD walk the same sequence of tile lengths (a round may leave some of them out)
    for x in range(8):
        seqs = [tuple(c for p, _, _, c in lists[w] if p >= 0) for w in range(x, 256, 8)]
        longest = max(seqs, key=len)
        for s in seqs:
            it = iter(longest)
            assert all(c in it for c in s), (x, s, longest)   # s is a subsequence of the longest list
