#!/usr/bin/env python3
"""Build-time check for the kernels of tile_f16_asm.h: their accumulators live in the accumulation registers
between hand-written assembly statements, so the compiler's own code must never touch those registers.

    check_asm_registers.py kernels_tile_asm.s

Reads the compiler's assembly listing of OUR translation unit (hipcc -S of kernels_tile_asm.hip) and fails if an
accumulation-register instruction or operand appears outside the ;;#ASMSTART ... ;;#ASMEND regions, or if a
kernel uses scratch memory.
"""
import re
import sys


def main(path):
    inside, bad = False, []
    for no, line in enumerate(open(path), 1):
        if "#ASMSTART" in line:
            inside = True
            continue
        if "#ASMEND" in line:
            inside = False
            continue
        code = line.split(";")[0]
        if not inside and re.search(r"v_accvgpr|v_mfma|\ba\[?\d", code):
            bad.append((no, line.strip()))
        m = re.match(r"\s*\.amdhsa_private_segment_fixed_size\s+(\d+)", line)
        if m and int(m.group(1)) != 0:
            bad.append((no, "kernel uses scratch memory: " + line.strip()))
    for no, text in bad[:20]:
        print(f"{path}:{no}: {text}", file=sys.stderr)
    if bad:
        sys.exit(f"{len(bad)} problem(s): the compiler touches accumulation registers (or spills) in an assembly-loop kernel")
    print(f"{path}: accumulation registers are only used inside the hand-written blocks; no scratch")


if __name__ == "__main__":
    main(sys.argv[1])
