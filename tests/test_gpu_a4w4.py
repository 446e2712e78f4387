"""MXFP4 (packed E2M1 + E8M0) on the GPU against the oracle: quantiser bit for bit, GEMM exact on the
general kernel and on integer inputs, |C - Cref| <= 1e-2*|Cref| + 1e-2 on the pipelined kernel (with the
same allowance for cancellation-dominated outputs as the MXFP8 tests: under 0.1%, each within 1e-4 of
sum|a||b|s of the float64 value)."""
import numpy as np
import pytest
import torch

import gcnasm_amd as g
from gpu_util import MFMA_ACC_ERR, dev

pytestmark = pytest.mark.gpu


def _x(rows, k, seed):
    rng = np.random.Generator(np.random.Philox(seed))
    x = rng.standard_normal((rows, k)).astype(np.float32)
    return x * np.exp2(rng.integers(-4, 5, (rows, k // 32))).repeat(32, axis=1).astype(np.float32)


def _exact(orc, qa, qb, ea, eb):
    A = orc.e2m1_decode_packed(qa).astype(np.float64) * np.exp2(ea.astype(np.float64) - 127).repeat(32, axis=1)
    B = orc.e2m1_decode_packed(qb).astype(np.float64) * np.exp2(eb.astype(np.float64) - 127).repeat(32, axis=1)
    return A @ B.T, np.abs(A) @ np.abs(B).T


@pytest.mark.parametrize("rows,k", [(1, 32), (37, 96), (256, 1024), (70, 7168)])
def test_quantiser_matches_oracle(orc, rows, k):
    x = _x(rows, k, 3 + rows)
    x[0, :32] = [6 * 2.0 ** -3] + [0] * 31                    # exactly a power of two times 6
    q, s = g.quantize_mxfp4(dev(x))
    qr, sr = orc.quantize_mxfp4(x)
    assert (s.cpu().numpy() == sr).all() and (q.cpu().numpy() == qr).all()
    qt, st = g.quantize_mxfp4(dev(x), tiled=True)
    assert torch.equal(qt, q) and (st.cpu().numpy() == orc.mx_tile_scales(sr)).all()


@pytest.mark.parametrize("shape", [(37, 53, 96), (64, 64, 224), (70, 40, 384)])       # k % 256 != 0: no MFMA kernel
def test_general_kernel_is_bit_exact(orc, shape):
    m, n, k = shape
    qa, ea = orc.quantize_mxfp4(_x(m, k, 11))
    qb, eb = orc.quantize_mxfp4(_x(n, k, 12))
    ref = orc.gemm_ref_mxfp4(qa, qb, ea, eb)
    got = g.gemm_a4w4(dev(qa), dev(qb), dev(ea), dev(eb), g.MX, c_dtype=g.FP32).cpu().numpy()
    assert (got == ref).all()
    ta, tb = g.mx_tile_scales(dev(ea)), g.mx_tile_scales(dev(eb))
    got = g.gemm_a4w4(dev(qa), dev(qb), ta, tb, g.MX_TILED, c_dtype=g.FP32).cpu().numpy()
    assert (got == ref).all()


# (the last two: short and wide with a long K loop, which the 128-tile kernel runs on 128 x 64 tiles)
@pytest.mark.parametrize("shape", [(256, 256, 512), (512, 256, 2048), (130, 270, 1024), (300, 520, 768),
                                   (200, 1088, 4096), (256, 320, 4352)])
def test_pipelined_kernel(orc, shape):
    m, n, k = shape
    qa, ea = orc.quantize_mxfp4(_x(m, k, 21 + m))
    qb, eb = orc.quantize_mxfp4(_x(n, k, 22 + n))
    ref = orc.gemm_ref_mxfp4(qa, qb, ea, eb)
    exact, mag = _exact(orc, qa, qb, ea, eb)
    ta, tb = g.mx_tile_scales(dev(ea)), g.mx_tile_scales(dev(eb))
    c32 = g.gemm_a4w4(dev(qa), dev(qb), ta, tb, c_dtype=g.FP32).cpu().numpy()
    assert (np.abs(c32 - exact) <= MFMA_ACC_ERR * mag + 1e-30).all()
    c = g.gemm_a4w4(dev(qa), dev(qb), ta, tb).float().cpu().numpy()
    miss = ~(np.abs(c - ref) <= 1e-2 * np.abs(ref) + 1e-2)
    assert miss.mean() <= 1e-3
    assert (np.abs(c - exact)[miss] <= MFMA_ACC_ERR * mag[miss] + 2.0 ** -8 * np.abs(exact)[miss]).all()


def test_scale_bytes_reach_the_right_lane_and_half(orc):
    """Distinct powers of two per (row, 32-block) on exactly representable operands: any mix-up of row,
    block, fragment half or op_sel byte changes the exact result."""
    m, n, k = 256, 512, 1024
    rng = np.random.Generator(np.random.Philox(9))
    qa = rng.integers(0, 256, (m, k // 2), dtype=np.uint8)
    qb = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    ea = (125 + (np.arange(m)[:, None] * 3 + np.arange(k // 32)[None, :]) % 4).astype(np.uint8)
    eb = (126 + (np.arange(n)[:, None] * 5 + np.arange(k // 32)[None, :] * 2) % 3).astype(np.uint8)
    exact, _ = _exact(orc, qa, qb, ea, eb)                     # sums of multiples of 2^-6 below 2^17: exact in fp32
    got = g.gemm_a4w4(dev(qa), dev(qb), g.mx_tile_scales(dev(ea)), g.mx_tile_scales(dev(eb)), c_dtype=g.FP32).cpu().numpy()
    assert (got == exact).all()


@pytest.mark.parametrize("shape", [(256, 256, 512), (130, 270, 1024), (300, 520, 768), (200, 1088, 4096), (256, 320, 4352),
                                   (1024, 2304, 256), (640, 4224, 1280)])
def test_row_major_scales_on_the_pipelined_kernel(orc, shape):
    """Row-major E8M0 scales (the quantiser's plain output) with k a multiple of 256 run on the 128-tile MFMA kernel, at
    any size: same bound against the float64 value as the tiled-scale path, same bits where that path runs the same
    kernel (up to two 128 x 128 tiles per compute unit)."""
    m, n, k = shape
    qa, ea = orc.quantize_mxfp4(_x(m, k, 31 + m))
    qb, eb = orc.quantize_mxfp4(_x(n, k, 32 + n))
    ref = orc.gemm_ref_mxfp4(qa, qb, ea, eb)
    exact, mag = _exact(orc, qa, qb, ea, eb)
    c32 = g.gemm_a4w4(dev(qa), dev(qb), dev(ea), dev(eb), g.MX, c_dtype=g.FP32)
    assert (np.abs(c32.cpu().numpy() - exact) <= MFMA_ACC_ERR * mag + 1e-30).all()
    if ((m + 127) // 128) * ((n + 127) // 128) <= 512:
        assert torch.equal(c32, g.gemm_a4w4(dev(qa), dev(qb), g.mx_tile_scales(dev(ea)), g.mx_tile_scales(dev(eb)), c_dtype=g.FP32))
    c = g.gemm_a4w4(dev(qa), dev(qb), dev(ea), dev(eb), g.MX).float().cpu().numpy()
    miss = ~(np.abs(c - ref) <= 1e-2 * np.abs(ref) + 1e-2)
    assert miss.mean() <= 1e-3
    assert (np.abs(c - exact)[miss] <= MFMA_ACC_ERR * mag[miss] + 2.0 ** -8 * np.abs(exact)[miss]).all()


@pytest.mark.parametrize("shape", [(256, 512, 1024), (100, 200, 256), (128, 1100, 4096), (384, 640, 2304)])
def test_row_major_scale_bytes_reach_the_right_lane_and_block(orc, shape):
    """Distinct powers of two per (row, 32-block) on exactly representable operands, row-major scales: any mix-up of
    row, block or byte changes the exact result."""
    m, n, k = shape
    rng = np.random.Generator(np.random.Philox(19 + m))
    qa = rng.integers(0, 256, (m, k // 2), dtype=np.uint8)
    qb = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    ea = (125 + (np.arange(m)[:, None] * 3 + np.arange(k // 32)[None, :]) % 4).astype(np.uint8)
    eb = (126 + (np.arange(n)[:, None] * 5 + np.arange(k // 32)[None, :] * 2) % 3).astype(np.uint8)
    exact, _ = _exact(orc, qa, qb, ea, eb)
    got = g.gemm_a4w4(dev(qa), dev(qb), dev(ea), dev(eb), g.MX, c_dtype=g.FP32).cpu().numpy()
    bad = np.argwhere(got != exact.astype(np.float32))
    assert bad.size == 0, f"{m}x{n}x{k}: {len(bad)} elements differ, first {bad[:4].tolist()}"


def test_full_size_8192(orc):
    m = n = k = 8192
    gen = torch.Generator(device="cuda"); gen.manual_seed(7)
    xa = torch.randn((m, k), generator=gen, device="cuda")
    xb = torch.randn((n, k), generator=gen, device="cuda")
    qa, ta = g.quantize_mxfp4(xa, tiled=True)
    qb, tb = g.quantize_mxfp4(xb, tiled=True)
    _, ea = g.quantize_mxfp4(xa[:8].contiguous())
    _, eb = g.quantize_mxfp4(xb)
    del xa, xb
    c = g.gemm_a4w4(qa, qb, ta, tb)
    ref = orc.gemm_ref_mxfp4(qa[:8].cpu().numpy(), qb.cpu().numpy(), ea.cpu().numpy(), eb.cpu().numpy())
    got = c[:8].float().cpu().numpy()
    assert (np.abs(got - ref) <= 1e-2 * np.abs(ref) + 1e-2).all()
    np.testing.assert_allclose(got, ref, rtol=2e-2, atol=2e-2 * np.abs(ref).max())
    # permuting the rows of A (with their scales) permutes the rows of C bit for bit
    perm = torch.randperm(m, generator=torch.Generator().manual_seed(3)).cuda()
    qa_p = qa[perm].contiguous()
    e_np = orc.mx_untile_scales(ta.cpu().numpy(), m, k)          # row-major scales of A, to permute and re-tile
    tp = g.mx_tile_scales(dev(e_np[perm.cpu().numpy()]))
    assert torch.equal(g.gemm_a4w4(qa_p, qb, tp, tb), c[perm])


# ---------------------------------------------------------------- flat (skinny-M) MXFP4 GEMM over pre-shuffled weights

def _flat(qa, qb, ea, eb, c_dtype=g.FP32):
    n = qb.shape[0]
    bs = g.preshuffle_b_device(dev(qb))                     # the packed weight bytes [N, K/2], shuffled as bytes
    c = g.flatmm_a4w4(dev(qa), bs, g.mx_tile_scales(dev(ea)), g.mx_tile_scales(dev(eb)), n, c_dtype=c_dtype)
    torch.cuda.synchronize()
    return c.float().cpu().numpy()


@pytest.mark.parametrize("shape", [(16, 256, 512), (16, 1024, 7168), (5, 48, 128), (33, 128, 384), (64, 4096, 1024), (1, 16, 128)])
def test_flat_against_the_oracle(orc, shape):
    m, n, k = shape
    qa, ea = orc.quantize_mxfp4(_x(m, k, 61 + m))
    qb, eb = orc.quantize_mxfp4(_x(n, k, 62 + n))
    want = orc.gemm_ref_mxfp4(qa, qb, ea, eb)
    exact, mag = _exact(orc, qa, qb, ea, eb)
    got = _flat(qa, qb, ea, eb)
    assert (np.abs(got - exact) <= MFMA_ACC_ERR * mag + 1e-30).all()
    got16 = _flat(qa, qb, ea, eb, g.BF16)
    miss = ~(np.abs(got16 - want) <= 1e-2 * np.abs(want) + 1e-2)
    assert miss.mean() <= 1e-3
    assert (np.abs(got16 - exact)[miss] <= MFMA_ACC_ERR * mag[miss] + 2.0 ** -8 * np.abs(exact)[miss]).all()


@pytest.mark.parametrize("case", range(24))
def test_flat_scale_bytes_reach_the_right_lane_and_block(orc, case):
    """Random E2M1 codes with a distinct power of two per (row, 32-block): every value is a multiple of 0.5 of
    magnitude <= 6 and the scales are 2^-1..2^1, so sums are exact in fp32 and any mix-up of row, block or the
    pair's byte changes the result."""
    r = np.random.default_rng(8000 + case)
    m = int(r.integers(1, 129))
    n = 16 * int(r.integers(1, 70))
    k = 128 * int(r.integers(1, 24))
    qa = r.integers(0, 256, (m, k // 2)).astype(np.uint8)
    qb = r.integers(0, 256, (n, k // 2)).astype(np.uint8)
    ea = r.integers(126, 129, (m, k // 32)).astype(np.uint8)
    eb = r.integers(126, 129, (n, k // 32)).astype(np.uint8)
    exact, _ = _exact(orc, qa, qb, ea, eb)
    got = _flat(qa, qb, ea, eb)
    bad = np.argwhere(got != exact.astype(np.float32))
    assert bad.size == 0, f"{m}x{n}x{k}: {len(bad)} elements differ, first {bad[:4].tolist()}"
    assert (_flat(qa, qb, ea, eb, g.BF16) == torch.from_numpy(exact.astype(np.float32)).to(torch.bfloat16).float().numpy()).all()


@pytest.mark.parametrize("m", [17, 32, 33, 48, 49, 64, 80, 128])
def test_flat_row_groups_four_weight_tiles(orc, m):
    """Enough weight tiles for four per workgroup (two past 48 rows), 1025 of them so that the last workgroup holds
    one; 2 / 3 / 4 groups of 16 rows share the pass over the weights."""
    r = np.random.default_rng(8700 + m)
    n, k = 16400, 384
    qa = r.integers(0, 256, (m, k // 2)).astype(np.uint8)
    qb = r.integers(0, 256, (n, k // 2)).astype(np.uint8)
    ea = r.integers(126, 129, (m, k // 32)).astype(np.uint8)
    eb = r.integers(126, 129, (n, k // 32)).astype(np.uint8)
    exact, _ = _exact(orc, qa, qb, ea, eb)
    got = _flat(qa, qb, ea, eb)
    bad = np.argwhere(got != exact.astype(np.float32))
    assert bad.size == 0, f"{m}x{n}x{k}: {len(bad)} elements differ, first {bad[:4].tolist()}"


@pytest.mark.parametrize("m", [1, 16, 33, 64, 100, 128])
@pytest.mark.parametrize("n", [144, 16400])
def test_skinny_gemm_on_row_major_weights(orc, m, n):
    """a4w4_gemm with at most 128 rows on row-major packed weights runs the flat kernel: exact, and the same bits
    as a4w4_flatmm on the shuffled weights."""
    r = np.random.default_rng(8900 + m + n)
    k = 384
    qa = r.integers(0, 256, (m, k // 2)).astype(np.uint8)
    qb = r.integers(0, 256, (n, k // 2)).astype(np.uint8)
    ea = r.integers(126, 129, (m, k // 32)).astype(np.uint8)
    eb = r.integers(126, 129, (n, k // 32)).astype(np.uint8)
    exact, _ = _exact(orc, qa, qb, ea, eb)
    ta, tb = g.mx_tile_scales(dev(ea)), g.mx_tile_scales(dev(eb))
    got = g.gemm_a4w4(dev(qa), dev(qb), ta, tb, c_dtype=g.FP32)
    torch.cuda.synchronize()
    bad = np.argwhere(got.cpu().numpy() != exact.astype(np.float32))
    assert bad.size == 0, f"{m}x{n}x{k}: {len(bad)} elements differ, first {bad[:4].tolist()}"
    assert torch.equal(got, g.flatmm_a4w4(dev(qa), g.preshuffle_b_device(dev(qb)), ta, tb, n, c_dtype=g.FP32))


def test_flat_rejects_what_it_cannot_run():
    qa = torch.zeros((16, 64), dtype=torch.uint8, device="cuda")
    bs = torch.zeros(16 * 64, dtype=torch.uint8, device="cuda")
    t = torch.full((1024,), 127, dtype=torch.uint8, device="cuda")
    assert g.flatmm_a4w4(qa, bs, t, t, 16).shape == (16, 16)
    with pytest.raises(g.A8W8Error, match="aligned"):
        g.flatmm_a4w4(torch.zeros((16, 64 + 8), dtype=torch.uint8, device="cuda")[:, :64], bs, t, t, 16)
    with pytest.raises(g.A8W8Error):
        g.flatmm_a4w4(torch.zeros((129, 64), dtype=torch.uint8, device="cuda"), bs, t, t, 16)
    with pytest.raises(g.A8W8Error):
        g.flatmm_a4w4(torch.zeros((16, 32), dtype=torch.uint8, device="cuda"), bs, t, t, 16)      # k = 64: not a whole block
