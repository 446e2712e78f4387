"""Seeded synthetic inputs for the five benchmark configurations (host side, numpy).

Quantisation uses the oracle's encoder, so this module is test infrastructure as well.
A is [M,K], B is [N,K] (row-major, i.e. the column-major K x N weight of the reference).
"""
import numpy as np

import oracle

SEED_BASE = 0xA8A80000
E4M3_MAX = 448.0


def _rng(seed):
    return np.random.Generator(np.random.Philox(seed))


def _q(x, scale):
    return oracle.encode((x / scale).astype(np.float32))


def per_tensor(m, n, k, seed=SEED_BASE + 1):
    r = _rng(seed)
    a = r.standard_normal((m, k), dtype=np.float32)
    b = r.standard_normal((n, k), dtype=np.float32)
    sa = np.float32(np.abs(a).max() / E4M3_MAX)
    sb = np.float32(np.abs(b).max() / E4M3_MAX)
    return _q(a, sa), _q(b, sb), np.array([sa], np.float32), np.array([sb], np.float32)


def row_col(m, n, k, seed=SEED_BASE + 2):
    r = _rng(seed)
    a = r.standard_normal((m, k), dtype=np.float32)
    b = r.standard_normal((n, k), dtype=np.float32)
    sa = (np.abs(a).max(axis=1) / E4M3_MAX).astype(np.float32)
    sb = (np.abs(b).max(axis=1) / E4M3_MAX).astype(np.float32)
    return _q(a, sa[:, None]), _q(b, sb[:, None]), sa, sb


def block_scaled(m, n, k, seed=SEED_BASE + 3):
    """A: 1x128 scales stored [K/128, M]; B: 128x128 scales stored [N/128, K/128]."""
    r = _rng(seed)
    a = r.standard_normal((m, k), dtype=np.float32)
    b = r.standard_normal((n, k), dtype=np.float32)
    sa = (np.abs(a.reshape(m, k // 128, 128)).max(axis=2) / E4M3_MAX).astype(np.float32)      # [M, K/128]
    sb = (np.abs(b.reshape(n // 128, 128, k // 128, 128)).max(axis=(1, 3)) / E4M3_MAX).astype(np.float32)
    qa = _q(a.reshape(m, k // 128, 128), sa[:, :, None]).reshape(m, k)
    qb = _q(b.reshape(n // 128, 128, k // 128, 128), sb[:, None, :, None]).reshape(n, k)
    return qa, qb, np.ascontiguousarray(sa.T), sb


def _mx_quant(x):
    rows, k = x.shape
    blk = x.reshape(rows, k // 32, 32)
    amax = np.abs(blk).max(axis=2)
    with np.errstate(divide="ignore"):
        e = np.ceil(np.log2(amax / E4M3_MAX))
    e = np.where(amax > 0, e, -127)
    e = np.clip(e, -127, 127).astype(np.int32)
    q = oracle.encode(np.ldexp(blk, -e[:, :, None]).astype(np.float32)).reshape(rows, k)
    return q, (e + 127).astype(np.uint8)


def mx(m, n, k, seed=SEED_BASE + 4):
    """E4M3 elements with one E8M0 exponent per 32 K-elements; values N(0,1)*2^U(-4,4) per block."""
    r = _rng(seed)
    out = []
    for rows in (m, n):
        x = r.standard_normal((rows, k), dtype=np.float32)
        x = x.reshape(rows, k // 32, 32) * np.exp2(r.uniform(-4, 4, (rows, k // 32, 1))).astype(np.float32)
        out.append(_mx_quant(x.reshape(rows, k).astype(np.float32)))
    (qa, ea), (qb, eb) = out
    return qa, qb, ea, eb


def small_ints(m, n, k, seed=7, lo=-4, hi=4):
    """Exact-integer operands (every product and partial sum is exact in fp32)."""
    r = _rng(seed)
    a = r.integers(lo, hi + 1, (m, k)).astype(np.float32)
    b = r.integers(lo, hi + 1, (n, k)).astype(np.float32)
    return oracle.encode(a), oracle.encode(b)


def reference_style(m, n, k, seed=11):
    """A~U[0,1), B~U[-.5,.5), scales~U[.8,1.2): the ranges of the reference harness."""
    r = _rng(seed)
    a = oracle.encode(r.uniform(0, 1, (m, k)).astype(np.float32))
    b = oracle.encode(r.uniform(-0.5, 0.5, (n, k)).astype(np.float32))
    sfa = r.uniform(0.8, 1.2, (k // 128, m)).astype(np.float32)
    sfb = r.uniform(0.8, 1.2, (n // 128, k // 128)).astype(np.float32)
    return a, b, sfa, sfb


def tolerance_ok(c, cref):
    """|C - Cref| <= 1e-2*|Cref| + 1e-2, the acceptance bound for GEMM outputs."""
    c = np.asarray(c, np.float32)
    cref = np.asarray(cref, np.float32)
    return np.abs(c - cref) <= 1e-2 * np.abs(cref) + 1e-2
