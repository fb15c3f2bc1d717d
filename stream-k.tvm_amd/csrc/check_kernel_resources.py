#!/usr/bin/env python3
"""Build-time check of the compiler's assembly listing of one translation unit (hipcc -save-temps).

    check_kernel_resources.py [--accumulation-registers] kernels_x.s

1. No kernel may use scratch memory (register spills: `.amdhsa_private_segment_fixed_size` > 0) unless its mangled
   name contains one of the patterns listed in scratch_allowed.txt (one per line: pattern, a tab or two spaces, the
   reason).
2. --accumulation-registers (the units of tile_f16_asm.h): their kernels keep the accumulators in the accumulation
   registers between hand-written assembly statements, so the compiler's own code must never touch those registers:
   no accumulation-register instruction or operand outside the ;;#ASMSTART ... ;;#ASMEND regions.
"""
import os
import re
import sys


def allowed_patterns():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "scratch_allowed.txt")
    out = []
    if os.path.exists(path):
        for line in open(path):
            line = line.strip()
            if line and not line.startswith("#"):
                out.append(re.split(r"\t|  +", line, maxsplit=1)[0])
    return out


def main(argv):
    check_acc = "--accumulation-registers" in argv
    path = [a for a in argv if not a.startswith("--")][0]
    allowed = allowed_patterns()
    inside, bad, kernel, spilled, listed = False, [], None, 0, 0
    for no, line in enumerate(open(path), 1):
        if "#ASMSTART" in line:
            inside = True
            continue
        if "#ASMEND" in line:
            inside = False
            continue
        m = re.match(r"\s*\.amdhsa_kernel\s+(\S+)", line)
        if m:
            kernel = m.group(1)
        code = line.split(";")[0]
        if check_acc and not inside and re.search(r"v_accvgpr|v_mfma|\ba\[?\d", code):
            bad.append((no, "accumulation register outside the hand-written blocks: " + line.strip()))
        m = re.match(r"\s*\.amdhsa_private_segment_fixed_size\s+(\d+)", line)
        if m and int(m.group(1)) != 0:
            spilled += 1
            if any(p in (kernel or "") for p in allowed):
                listed += 1
            else:
                bad.append((no, f"kernel uses {m.group(1)} bytes of scratch memory per lane and is not in scratch_allowed.txt: {kernel}"))
    for no, text in bad[:20]:
        print(f"{path}:{no}: {text}", file=sys.stderr)
    if bad and "--warn-only" in argv:     # (for experiments: make CHECK_EXTRA=--warn-only)
        print(f"{len(bad)} problem(s) in {path}: ignored", file=sys.stderr)
        return
    if bad:
        sys.exit(f"{len(bad)} problem(s) in {path}")
    acc = "; accumulation registers only inside the hand-written blocks" if check_acc else ""
    print(f"{os.path.basename(path)}: {spilled - listed} unlisted scratch users ({listed} listed){acc}")


if __name__ == "__main__":
    main(sys.argv[1:])
