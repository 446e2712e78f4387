#!/usr/bin/env python3
"""Build-time check of the compiler's output for the four-wave GEMM kernels.

Those kernels keep their accumulators in registers a[0:255] that only their own assembly statements
name.  That is sound as long as the compiler places nothing of its own there and spills nothing:
this script reads the device assembly of the library and fails the build otherwise.
Usage: check_isa.py <device .s file>
"""
import re
import sys


def main(path):
    text = open(path).read()
    funcs = re.split(r"\n(?=_Z\w+:)", text)
    checked = 0
    for f in funcs:
        name = f.split(":", 1)[0]
        if "gemm_a8w8_wide" not in name:
            continue
        checked += 1
        mfma = reads = 0
        for line in f.split("\n"):
            ins = line.split(";", 1)[0].strip()
            if not ins or ins.startswith("."):
                continue
            op = ins.split()[0]
            if op.startswith("v_mfma"):
                mfma += 1
                continue
            if op == "v_accvgpr_read_b32":
                reads += 1
                continue
            if op.startswith("scratch_"):
                sys.exit(f"{name}: spills to scratch: {ins}")
            if op.startswith("v_accvgpr"):
                sys.exit(f"{name}: compiler-made accumulator register traffic: {ins}")
            if re.search(r"\ba(\[\d+(:\d+)?\]|\d+)\b", ins.split(None, 1)[1] if " " in ins else ""):
                sys.exit(f"{name}: accumulator register used outside the kernel's own statements: {ins}")
        if mfma == 0 or reads == 0:
            sys.exit(f"{name}: expected MFMAs and accumulator reads, found {mfma} and {reads}")
    if checked == 0:
        sys.exit("no four-wave kernel found in " + path)
    print(f"four-wave kernels: {checked} checked, accumulator registers untouched by the compiler, no scratch")


if __name__ == "__main__":
    main(sys.argv[1])
