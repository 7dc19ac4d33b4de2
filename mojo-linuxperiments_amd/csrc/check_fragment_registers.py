#!/usr/bin/env python3
"""Build check for the hand-scheduled GEMM kernels: usage  check_fragment_registers.py FILE.s KERNEL_SUBSTRING [N_RANGES]

The kernels read their matrix-instruction operands ("fragments") from LDS with ds_read_b128 inside asm statements and
wait for them with hand-counted s_waitcnt.  The compiler does not know that such a register holds its value only
later, so it must never copy one: a v_mov out of a fragment register between the read and the wait would copy what
the register held before.  This script reads the compiler's assembly of the kernels whose names contain
KERNEL_SUBSTRING and stops the build when
  - a register move (v_mov_b32, v_accvgpr_write_b32, v_swap_b32) takes a fragment register as its source, or
  - N_RANGES is given and the ds_read_b128 instructions of a kernel write another number of distinct register
    ranges (a fragment must live in the same registers in every copy the compiler makes of the stage code: it
    peels or duplicates loops as it sees fit, and a fragment that changed registers between two copies would have
    to be moved)."""
import re
import sys


def kernels(text, sub):
    out = {}
    for m in re.finditer(r"^(\w+):[^\n]*\n(.*?)^\.Lfunc_end\d+:", text, re.S | re.M):
        if sub in m.group(1) and "v_mfma" in m.group(2):
            out[m.group(1)] = m.group(2)
    return out


def main():
    path, sub = sys.argv[1], sys.argv[2]
    want = int(sys.argv[3]) if len(sys.argv) > 3 else 0
    ks = kernels(open(path).read(), sub)
    if not ks:
        sys.exit("check_fragment_registers: no kernel *%s* with matrix instructions in %s" % (sub, path))
    bad = []
    for name, body in ks.items():
        ranges = set((int(a), int(b)) for a, b in re.findall(r"ds_read_b128 v\[(\d+):(\d+)\]", body))
        frag = set()
        for a, b in ranges:
            frag.update(range(a, b + 1))
        if want and len(ranges) != want:
            bad.append("%s: ds_read_b128 writes %d distinct register ranges, expected %d" % (name, len(ranges), want))
        if len(frag) != 4 * len(ranges):
            bad.append("%s: fragment register ranges overlap: %s" % (name, sorted(ranges)))
        for n, line in enumerate(body.split("\n")):
            m = re.match(r"\s*(v_mov_b32\w*|v_accvgpr_write_b32|v_swap_b32)\s+(\S+),\s*(\S+)", line)
            if not m:
                continue
            srcs = [m.group(3)] + ([m.group(2)] if m.group(1) == "v_swap_b32" else [])
            for s in srcs:
                r = re.match(r"v(\d+)\b", s)
                if r and int(r.group(1)) in frag:
                    bad.append("%s: line %d copies fragment register %s: %s" % (name, n, s, line.strip()))
    if bad:
        sys.exit("check_fragment_registers:\n  " + "\n  ".join(bad))
    print("check_fragment_registers: %d kernel(s) *%s*: no move out of a fragment register%s"
          % (len(ks), sub, ", %d fragment ranges each" % want if want else ""))


if __name__ == "__main__":
    main()
