#!/usr/bin/env python3
"""Build-time checks of the compiler's output.

Every kernel: a 16-byte (or 12-byte) buffer store (the C tiles' stores) reads its data registers for a few cycles after it
issues, so nothing may write them in the two issue slots behind it: the first write to one of them has to come after the
two idle cycles that store_c_16 (a8w8_device.hpp) puts behind the store, or after at least two other instructions.

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


def registers(operand):
    """The vector registers an operand names: 'v7' or 'v[4:7]' (anything else: none)."""
    m = re.fullmatch(r"v(\d+)", operand.strip())
    if m:
        return {int(m.group(1))}
    m = re.fullmatch(r"v\[(\d+):(\d+)\]", operand.strip())
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    return set()


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
                data = registers(ins.split(None, 1)[1].split(",")[0])
                # walk on until the idle cycles (or two other instructions) have passed; nothing before that may write the data
                slots = 0
                for nxt in seq[i + 1:i + 4]:
                    if nxt == "s_nop 1" or slots >= 2:
                        break
                    if nxt.startswith("s_nop"):
                        slots += 1 + int(nxt.split()[1])
                        continue
                    if nxt.endswith(":") or nxt.startswith("s_cbranch") or nxt.startswith("s_branch") or nxt.startswith("s_endpgm"):
                        sys.exit(f"{name}: control flow directly behind a 16-byte buffer store: {ins} / {nxt}")
                    parts = nxt.split(None, 1)
                    written = registers(parts[1].split(",")[0]) if len(parts) > 1 and not parts[0].startswith(("buffer_store", "global_store", "ds_write", "s_")) else set()
                    if written & data:
                        sys.exit(f"{name}: the data registers of a 16-byte buffer store are written directly behind it: {ins} / {nxt}")
                    slots += 1
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
    print(f"16-byte buffer stores: {stores} checked, none with a write to its data registers in the two slots behind it")


if __name__ == "__main__":
    main(sys.argv[1], "--no-stores-ok" in sys.argv[2:])
