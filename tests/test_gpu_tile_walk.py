"""More tiles than compute units, with ragged edges: one workgroup of the persistent GEMM kernels walks
several tiles, interior ones (written out piece by piece behind the next MFMAs) and edge ones
(bounds-checked epilogue) in every order.  Operands are small integers and scales powers of two, so
every partial sum is exact in fp32 and the result must match bit for bit; the expected value comes from
a float64 matrix product of the decoded operands (exact for these inputs)."""
import numpy as np
import pytest
import torch

import datagen
import gcnasm_amd as g
from gpu_util import dev

pytestmark = pytest.mark.gpu

SHAPE = (4389, 4229, 512)        # 18 x 17 = 306 tiles of 256 x 256 on 256 compute units, two K-step pairs


def _exact(orc, a, b):
    return orc.decode(a).astype(np.float64) @ orc.decode(b).astype(np.float64).T


def _pow2(r, n, lo=-3, hi=3):
    return np.exp2(r.integers(lo, hi + 1, n)).astype(np.float32)


def _check(c, want, what):
    got = c.float().cpu().numpy() if c.dtype != torch.float32 else c.cpu().numpy()
    if c.dtype == torch.bfloat16:
        want = torch.from_numpy(want.astype(np.float32)).to(torch.bfloat16).float().numpy()
    bad = np.argwhere(got != want.astype(np.float32))
    assert bad.size == 0, f"{what}: {len(bad)} elements differ, first {bad[:4].tolist()}"


@pytest.mark.parametrize("c_dtype", [g.BF16, g.FP32])
def test_per_tensor_and_rowcol(orc, c_dtype):
    m, n, k = SHAPE
    a, b = datagen.small_ints(m, n, k, seed=71)
    exact = _exact(orc, a, b)
    r = np.random.default_rng(72)
    sa, sb = np.array([0.5], np.float32), np.array([4.0], np.float32)
    args = g.raw_gemm_args(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, m, n, k, g.TENSOR)
    assert g.kernel_name(args) == "gemm_a8w8_wide"
    _check(g.gemm(dev(a), dev(b), dev(sa), dev(sb), g.TENSOR, c_dtype=c_dtype), exact * 2.0, "per-tensor")
    sa, sb = _pow2(r, m), _pow2(r, n)
    _check(g.gemm(dev(a), dev(b), dev(sa), dev(sb), g.ROWCOL, c_dtype=c_dtype),
           exact * sa[:, None].astype(np.float64) * sb[None, :], "row/col")


def test_rowcol_batched(orc):
    batch, m, n, k = 5, 2100, 1900, 256          # 9 x 8 x 5 = 360 work items, one K-step pair each
    per = [datagen.small_ints(m, n, k, seed=80 + i) for i in range(batch)]
    a = np.stack([p[0] for p in per])
    b = np.stack([p[1] for p in per])
    r = np.random.default_rng(81)
    sa = np.stack([_pow2(r, m) for _ in range(batch)])
    sb = np.stack([_pow2(r, n) for _ in range(batch)])
    c = g.gemm(dev(a), dev(b), dev(sa), dev(sb), g.ROWCOL, c_dtype=g.FP32)
    for i in range(batch):
        want = _exact(orc, a[i], b[i]) * sa[i][:, None].astype(np.float64) * sb[i][None, :]
        _check(c[i], want, f"batch entry {i}")


@pytest.mark.parametrize("c_dtype", [g.BF16, g.FP32])
def test_tiled_mx(orc, c_dtype):
    m, n, k = SHAPE
    a, b = datagen.small_ints(m, n, k, seed=73)
    r = np.random.default_rng(74)
    ea = r.integers(125, 130, (m, k // 32)).astype(np.uint8)       # 2^-2..2^2: sums stay exact in fp32
    eb = r.integers(125, 130, (n, k // 32)).astype(np.uint8)
    A = orc.decode(a).astype(np.float64) * np.repeat(np.exp2(ea.astype(np.float64) - 127), 32, axis=1)
    B = orc.decode(b).astype(np.float64) * np.repeat(np.exp2(eb.astype(np.float64) - 127), 32, axis=1)
    ta, tb = g.mx_tile_scales_ab(dev(ea), dev(eb))
    _check(g.gemm(dev(a), dev(b), ta, tb, g.MX_TILED, c_dtype=c_dtype), A @ B.T, "tiled MX")


def test_bf16_operands():
    m, n, k = 4389, 4229, 256
    gen = torch.Generator(device="cuda"); gen.manual_seed(75)
    a = torch.randint(-8, 9, (m, k), generator=gen, device="cuda").to(torch.bfloat16)
    b = torch.randint(-8, 9, (n, k), generator=gen, device="cuda").to(torch.bfloat16)
    want = (a.double() @ b.double().T).float()
    assert torch.equal(g.gemm_a16w16(a, b, c_dtype=g.FP32), want)
    assert torch.equal(g.gemm_a16w16(a, b), want.to(torch.bfloat16))


def test_mxfp4_operands(orc):
    m, n, k = 4389, 4229, 512
    r = np.random.default_rng(76)
    # E2M1 codes: every value a multiple of 0.5 with magnitude <= 6, block scales 2^-1..2^1: sums stay exact in fp32
    qa = r.integers(0, 256, (m, k // 2)).astype(np.uint8)
    qb = r.integers(0, 256, (n, k // 2)).astype(np.uint8)
    ea = r.integers(126, 129, (m, k // 32)).astype(np.uint8)
    eb = r.integers(126, 129, (n, k // 32)).astype(np.uint8)
    A = orc.e2m1_decode_packed(qa).astype(np.float64) * np.repeat(np.exp2(ea.astype(np.float64) - 127), 32, axis=1)
    B = orc.e2m1_decode_packed(qb).astype(np.float64) * np.repeat(np.exp2(eb.astype(np.float64) - 127), 32, axis=1)
    ta, tb = g.mx_tile_scales_ab(dev(ea), dev(eb))
    c = g.gemm_a4w4(dev(qa), dev(qb), ta, tb, c_dtype=g.FP32)
    _check(c, A @ B.T, "MXFP4")
