#!/usr/bin/env python3
"""Build-time checks of the compiler's output.

Every kernel: a 16-byte (or 12-byte) buffer store (the C tiles' stores) is followed, before anything that writes a vector
register, by the two idle cycles that keep the next write to its data registers at a distance (store_c_16 in
a8w8_device.hpp).

The four-wave GEMM kernels:

Those kernels keep their accumulators in registers a[0:255] that only their own assembly statements
name.  That is sound as long as the compiler places nothing of its own there and spills nothing:
this script reads the device assembly of the library and fails the build otherwise.
Usage: check_isa.py <device .s file> [--no-stores-ok]     (the option: for measurement builds that leave the stores out)
"""
import re
import sys


def instructions(func):
    for line in func.split("\n"):
        ins = line.split(";", 1)[0].strip()
        if ins and not ins.startswith(".") and not ins.endswith(":"):
            yield ins


def main(path, no_stores_ok=False):
    text = open(path).read()
    funcs = re.split(r"\n(?=_Z\w+:)", text)
    checked = stores = 0
    for f in funcs:
        name = f.split(":", 1)[0]
        seq = list(instructions(f))
        for i, ins in enumerate(seq):
            # every buffer store of more than 64 bits (should the compiler ever split 16 bytes into 12 + 4, the 12-byte
            # part is held to the same rule)
            if ins.startswith("buffer_store_dwordx4") or ins.startswith("buffer_store_dwordx3"):
                stores += 1
                # nothing that could write a vector register may come between the store and its idle cycles
                j = i + 1
                while j < len(seq) and seq[j] != "s_nop 1" and (seq[j].startswith("s_") or seq[j].startswith("v_readlane_b32") or
                                                                 seq[j].startswith("v_readfirstlane_b32")):
                    j += 1
                if j >= len(seq) or seq[j] != "s_nop 1":
                    sys.exit(f"{name}: 16-byte buffer store without the idle cycles behind it: {ins} / {seq[j] if j < len(seq) else ''}")
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
    if stores == 0 and not no_stores_ok:
        sys.exit("no 16-byte buffer store found in " + path)
    print(f"four-wave kernels: {checked} checked, accumulator registers untouched by the compiler, no scratch")
    print(f"16-byte buffer stores: {stores} checked, each followed by its idle cycles")


if __name__ == "__main__":
    main(sys.argv[1], "--no-stores-ok" in sys.argv[2:])
