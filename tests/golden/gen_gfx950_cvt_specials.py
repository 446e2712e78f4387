#!/usr/bin/env python3
"""Records what v_cvt_pk_fp8_f32 returns on a gfx950 device for special and out-of-range inputs.

The reference's conversion helpers call the instruction through its builtin
(cvt_fp8/test.cpp:37, pk_cvt/test.cpp:242-243) and print, never assert, its results, so the
instruction itself is the authority for NaN, Inf and overflow.  This script feeds the inputs
below to the instruction (through the library's a8w8_cvt_f32_to_e4m3, OCP dialect, which issues
exactly that builtin) without and with the +-240 clamp and prints one line per input:

    f32_bits  code_unclamped  code_clamp240

Run on a GPU box:  python tests/golden/gen_gfx950_cvt_specials.py > gfx950_cvt_pk_fp8_specials.txt
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))

BITS = [0x7f800000, 0xff800000, 0x7fc00000, 0xffc00000, 0x7f800001, 0xff800001, 0x7fffffff,
        0x7f7fffff, 0xff7fffff]
VALUES = [1e9, -1e9, 449, -449, 448, -448, 464, -464, 465, -465, 480, -480, 241, -241, 240, -240, 248, 256,
          1e-30, -1e-30, 2.0 ** -10, 2.0 ** -11]


def main():
    import torch
    import gcnasm_amd as g
    x = np.concatenate([np.array(BITS, np.uint32).view(np.float32), np.array(VALUES, np.float32)])
    n = x.size
    x = np.concatenate([x, np.zeros((-n) % 4, np.float32)])
    t = torch.from_numpy(x).cuda()
    plain = g.cvt_f32_to_e4m3(t, 0, clamp240=False).cpu().numpy()
    clamped = g.cvt_f32_to_e4m3(t, 0, clamp240=True).cpu().numpy()
    print("# f32_bits code_unclamped code_clamp240   (v_cvt_pk_fp8_f32 on gfx950, OCP E4M3)")
    for b, p, c in zip(x.view(np.uint32)[:n], plain, clamped):
        print(f"{int(b):08x} {int(p):02x} {int(c):02x}")


if __name__ == "__main__":
    main()
