#!/usr/bin/env python3
"""Build-time check of the register contract of the kernels whose accumulators are numbered by hand.

Reads the remarks hipcc prints with -Rpass-analysis=kernel-resource-usage (a file) and fails the build when a kernel
whose mangled name contains NAME breaks one of the given limits, e.g.

    check_kernel_resources.py gemm_list.remarks k_w8a8_list vgprs=256 agprs=0 scratch=0 vgpr_spill=0 sgpr_spill=0 occupancy=2

Keys: vgprs / agprs (exact, or `vgprs<=64`), scratch, vgpr_spill, sgpr_spill (exact), occupancy (exact).
A hand-numbered register that the compiler also used (a spill, a split live range) would give wrong sums with no
error at run time; this is where such a build stops.
"""
import re
import sys

KEYS = {
    "vgprs": r"\bVGPRs: (\d+)",
    "agprs": r"\bAGPRs: (\d+)",
    "scratch": r"ScratchSize \[bytes/lane\]: (\d+)",
    "vgpr_spill": r"VGPRs Spill: (\d+)",
    "sgpr_spill": r"SGPRs Spill: (\d+)",
    "occupancy": r"Occupancy \[waves/SIMD\]: (\d+)",
}


def main(argv):
    if len(argv) < 4:
        print(__doc__)
        return 2
    text = open(argv[1]).read()
    name = argv[2]
    blocks = re.split(r"Function Name: ", text)[1:]
    mine = [b for b in blocks if name in b.split()[0]]
    if not mine:
        print("check_kernel_resources: no kernel named *%s* in %s" % (name, argv[1]))
        return 1
    bad = 0
    for b in mine:
        fn = b.split()[0]
        for cond in argv[3:]:
            m = re.match(r"(\w+)(<=|=)(\d+)$", cond)
            if not m or m.group(1) not in KEYS:
                print("check_kernel_resources: bad condition %r" % cond)
                return 2
            key, op, want = m.group(1), m.group(2), int(m.group(3))
            got = re.search(KEYS[key], b)
            if not got:
                print("check_kernel_resources: %s: no %s remark" % (fn, key))
                bad += 1
                continue
            v = int(got.group(1))
            ok = v <= want if op == "<=" else v == want
            if not ok:
                print("check_kernel_resources: %s: %s is %d, must be %s%d" % (fn, key, v, op, want))
                bad += 1
    if not bad:
        print("check_kernel_resources: %d kernel(s) *%s* within %s" % (len(mine), name, " ".join(argv[3:])))
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
