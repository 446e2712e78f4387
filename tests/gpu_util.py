"""Helpers for the GPU parity tests: move numpy inputs to the card, call the C ABI through
the gcnasm_amd binding, bring results back as fp32 numpy."""
import numpy as np
import torch

import gcnasm_amd as g


def dev(x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def run_gemm(a, b, sfa, sfb, mode, c_dtype=g.BF16):
    c = g.gemm(dev(a), dev(b), dev(sfa), dev(sfb), mode, c_dtype=c_dtype)
    torch.cuda.synchronize()
    return c.float().cpu().numpy()


def run_flatmm(a, bshuf, sfa, sfb, n, mode=g.ROWCOL, c_dtype=g.BF16):
    c = g.flatmm(dev(a), dev(bshuf), dev(sfa), dev(sfb), n, scale_mode=mode, c_dtype=c_dtype)
    torch.cuda.synchronize()
    return c.float().cpu().numpy()


MFMA_ACC_ERR = 1e-4   # measured bound of the gfx950 FP8 MFMA's internal accumulation error / sum|a||b|s


def assert_close(c, cref, what="", exact=None, mag=None):
    """|C - Cref| <= 1e-2*|Cref| + 1e-2 (bf16 output, fp32 accumulation) against the CPU reference.

    The FP8 MFMA aligns the 128 products of one instruction to their largest exponent and
    drops what falls below 24 bits, so its sums carry an error of up to ~5e-5 of sum|a||b|s
    (measured; sequential fp32 on the CPU has ~4e-7).  On the wide-range MX inputs that
    exceeds the 1e-2 absolute term for the few outputs that cancel to almost zero.  When the
    float64 value `exact` and `mag` = sum|a||b|s are given, elements that miss the bound may be
    at most 0.1% of the output and each must lie within MFMA_ACC_ERR*mag (+ bf16 rounding) of
    the float64 value; without them every element must meet the bound."""
    c = np.asarray(c, np.float32)
    cref = np.asarray(cref, np.float32)
    miss = ~(np.abs(c - cref) <= 1e-2 * np.abs(cref) + 1e-2)
    if exact is not None and miss.any():
        ex = np.asarray(exact, np.float64)
        assert miss.mean() <= 1e-3, f"{what}: {miss.sum()} of {c.size} outside tolerance"
        miss &= ~(np.abs(c - ex) <= MFMA_ACC_ERR * mag + 2.0 ** -8 * np.abs(ex))
    bad = np.argwhere(miss)
    assert bad.size == 0, (f"{what}: {len(bad)} of {c.size} outside tolerance, first {bad[:3].tolist()}, "
                           f"got {c[tuple(bad[0])]} want {cref[tuple(bad[0])]}")


def exact64(orc, a, b, sfa, sfb, mode):
    """float64 evaluation of the GEMM (exact up to 1e-16 relative) and of sum |a||b|scale,
    the natural yardstick for fp32 accumulation error."""
    A = orc.decode(a).astype(np.float64)
    B = orc.decode(b).astype(np.float64)
    m, k = A.shape
    n = B.shape[0]
    if mode == g.TENSOR:
        s = float(sfa[0]) * float(sfb[0])
        return (A @ B.T) * s, (np.abs(A) @ np.abs(B).T) * s
    if mode == g.ROWCOL:
        s = sfa.astype(np.float64)[:, None] * sfb.astype(np.float64)[None, :]
        return (A @ B.T) * s, (np.abs(A) @ np.abs(B).T) * s
    gk = 128 if mode == g.BLOCK else 32
    out = np.zeros((m, n))
    mag = np.zeros((m, n))
    for gi in range(k // gk):
        sl = slice(gi * gk, (gi + 1) * gk)
        if mode == g.BLOCK:
            s = sfa[gi].astype(np.float64)[:, None] * np.repeat(sfb[:, gi].astype(np.float64), 128)[None, :]
        else:
            s = np.exp2(sfa[:, gi].astype(np.float64) - 127)[:, None] * np.exp2(sfb[:, gi].astype(np.float64) - 127)[None, :]
        out += (A[:, sl] @ B[:, sl].T) * s
        mag += (np.abs(A[:, sl]) @ np.abs(B[:, sl]).T) * s
    return out, mag


def assert_fp32_accurate(got, exact, mag, what=""):
    """fp32 output against the float64 value: error within MFMA_ACC_ERR of sum|a||b|scale, the
    accumulation accuracy of the matrix cores; far tighter than bf16 rounding, so a misplaced
    scale or operand cannot hide in it."""
    err = np.abs(np.asarray(got, np.float64) - exact)
    bound = MFMA_ACC_ERR * mag + 1e-30
    bad = np.argwhere(~(err <= bound))
    assert bad.size == 0, f"{what}: {len(bad)} of {err.size} beyond fp32 accumulation error, first {bad[:3].tolist()}"
