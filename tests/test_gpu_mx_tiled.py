"""Tiled MX scale layout on the GPU: the re-ordering kernel and the quantiser's tiled output are
bit-exact against the oracle's walk over the layout, and a8w8_gemm with tiled scales returns what
the oracle's MX GEMM returns for the row-major scales (tolerance |C - Cref| <= 1e-2*|Cref| + 1e-2,
bit-exact on integer inputs)."""
import numpy as np
import pytest
import torch

import datagen
import gcnasm_amd as g
from gpu_util import assert_close, assert_fp32_accurate, dev, exact64

pytestmark = pytest.mark.gpu


def _tiled_gemm(a, b, ea, eb, c_dtype=g.BF16):
    ta, tb = g.mx_tile_scales(dev(ea)), g.mx_tile_scales(dev(eb))
    c = g.gemm(dev(a), dev(b), ta, tb, g.MX_TILED, c_dtype=c_dtype)
    torch.cuda.synchronize()
    return c.float().cpu().numpy()


@pytest.mark.parametrize("rows,k", [(64, 512), (256, 1024), (100, 384), (1, 32), (513, 7168), (70, 96)])
def test_tile_scales_kernel_matches_oracle(orc, rows, k):
    rng = np.random.Generator(np.random.Philox(rows * 7 + k))
    sf = rng.integers(0, 255, (rows, k // 32), dtype=np.uint8)
    got = g.mx_tile_scales(dev(sf)).cpu().numpy()
    want = orc.mx_tile_scales(sf)
    assert got.size == g.mx_tiled_bytes(rows, k) == want.size
    assert (got == want).all()
    # a row stride larger than the row (a view into a wider scale matrix)
    wide = rng.integers(0, 255, (rows, k // 32 + 5), dtype=np.uint8)
    got = g.mx_tile_scales(dev(wide)[:, : k // 32]).cpu().numpy()
    assert (got == orc.mx_tile_scales(wide[:, : k // 32])).all()


def test_both_arrays_in_one_launch(orc):
    rng = np.random.Generator(np.random.Philox(99))
    ea = rng.integers(0, 255, (130, 24), dtype=np.uint8)
    eb = rng.integers(0, 255, (520, 24), dtype=np.uint8)
    ta, tb = g.mx_tile_scales_ab(dev(ea), dev(eb))
    assert (ta.cpu().numpy() == orc.mx_tile_scales(ea)).all()
    assert (tb.cpu().numpy() == orc.mx_tile_scales(eb)).all()


@pytest.mark.parametrize("rows,k", [(128, 512), (70, 384), (300, 1024)])
def test_quantize_writes_the_tiled_layout(orc, rows, k):
    rng = np.random.Generator(np.random.Philox(41 + rows))
    x = (rng.standard_normal((rows, k)) * np.exp2(rng.integers(-6, 6, (rows, k // 32)).repeat(32, axis=1))).astype(np.float32)
    q0, s0 = g.quantize(dev(x), g.MX)
    q1, s1 = g.quantize(dev(x), g.MX_TILED)
    assert torch.equal(q0, q1)
    assert (s1.cpu().numpy() == orc.mx_tile_scales(s0.cpu().numpy())).all()


@pytest.mark.parametrize("shape", [(256, 256, 256), (512, 256, 1024), (130, 270, 768), (256, 512, 2048), (64, 64, 512),
                                   (70, 40, 384), (64, 64, 128), (2304, 2048, 256), (1300, 4000, 512), (2100, 2300, 384), (2304, 4096, 256), (2100, 4500, 384)])
def test_gemm_with_tiled_scales(orc, shape):
    """Up to 128 rows: the flat kernel.  At most 512 tiles of 128 x 128, or an odd number of K steps: the 128-tile kernel;
    otherwise the four-wave kernel."""
    m, n, k = shape
    a, b, ea, eb = datagen.mx(m, n, k, seed=1500 + m + k)
    args = g.raw_gemm_args(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, m, n, k, g.MX_TILED)
    workgroups128 = -(-m // 128) * -(-n // 128)
    flat = m <= 128 and n % 16 == 0 and k % 64 == 0          # skinny: the flat kernel, also on row-major weights
    assert g.kernel_name(args) == ("flatmm_a8w8" if flat else "gemm_a8w8_wide" if workgroups128 > 512 and k % 256 == 0 else "gemm_a8w8_tile128")
    want = orc.gemm_ref(a, b, ea, eb, orc.MX)
    exact, mag = exact64(orc, a, b, ea, eb, g.MX)
    assert_close(_tiled_gemm(a, b, ea, eb), want, f"mx tiled {shape}", exact=exact, mag=mag)
    assert_fp32_accurate(_tiled_gemm(a, b, ea, eb, g.FP32), exact, mag)


def test_tiled_scale_bytes_reach_the_right_lane_and_step(orc):
    """Each (row, 32-block) gets a distinct power of two and the inputs are small integers, so any
    mix-up of row, block, K step or op_sel byte changes the exact result."""
    m, n, k = 256, 512, 1024
    a, b = datagen.small_ints(m, n, k, seed=78, lo=-2, hi=2)
    ea = (125 + (np.arange(m)[:, None] * 3 + np.arange(k // 32)[None, :]) % 4).astype(np.uint8)
    eb = (126 + (np.arange(n)[:, None] * 5 + np.arange(k // 32)[None, :] * 2) % 3).astype(np.uint8)
    want = orc.gemm_ref(a, b, ea, eb, orc.MX)
    assert (_tiled_gemm(a, b, ea, eb, g.FP32) == want).all()


@pytest.mark.parametrize("shape", [(37, 53, 96), (70, 40, 352), (300, 270, 32)])
def test_tiled_scales_on_the_general_kernel(orc, shape):
    """k % 128 != 0 takes the general kernel, which follows the oracle's order of operations: bit-exact."""
    m, n, k = shape
    a, b, ea, eb = datagen.mx(m, n, k, seed=1600 + k)
    args = g.raw_gemm_args(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, m, n, k, g.MX_TILED)
    assert g.kernel_name(args) == "gemm_a8w8_general"
    want = orc.gemm_ref(a, b, ea, eb, orc.MX)
    assert (_tiled_gemm(a, b, ea, eb, g.FP32) == want).all()


def test_tiled_equals_row_major_bit_for_bit_at_full_size(orc):
    """8192^3: the tiled-scale GEMM reproduces the row-major-scale GEMM exactly (same products, same
    accumulation order), so every check made on one holds for the other."""
    m = n = k = 8192
    a, b, ea, eb = datagen.mx(m, n, k)
    da, db, dea, deb = dev(a), dev(b), dev(ea), dev(eb)
    c = g.gemm(da, db, dea, deb, g.MX)
    ct = g.gemm(da, db, g.mx_tile_scales(dea), g.mx_tile_scales(deb), g.MX_TILED)
    assert torch.equal(c, ct)


def test_batched_and_more_tiles_than_compute_units(orc):
    batch, m, n, k = 3, 300, 520, 512
    per = [datagen.mx(m, n, k, seed=1950 + i) for i in range(batch)]
    a, b, ea, eb = (np.stack([p[i] for p in per]) for i in range(4))
    ta = torch.stack([g.mx_tile_scales(dev(ea[i])) for i in range(batch)])
    tb = torch.stack([g.mx_tile_scales(dev(eb[i])) for i in range(batch)])
    c = g.gemm(dev(a), dev(b), ta, tb, g.MX_TILED, c_dtype=g.FP32).cpu().numpy()
    for i in range(batch):
        ref = orc.gemm_ref(a[i], b[i], ea[i], eb[i], orc.MX)
        np.testing.assert_allclose(c[i], ref, rtol=2e-3, atol=2e-3 * np.abs(ref).max())
    m = n = 4352   # 17 x 17 tiles on 256 CUs
    a, b = datagen.small_ints(m, n, 512, seed=1903, lo=-2, hi=2)
    ea = (126 + (np.arange(m)[:, None] + np.arange(16)[None, :]) % 3).astype(np.uint8)
    eb = (126 + (np.arange(n)[:, None] * 2 + np.arange(16)[None, :]) % 3).astype(np.uint8)
    sa = np.exp2(ea.astype(np.float32) - 127).repeat(32, axis=1)
    sb = np.exp2(eb.astype(np.float32) - 127).repeat(32, axis=1)
    want = torch.from_numpy(orc.decode(a) * sa).cuda() @ torch.from_numpy(orc.decode(b) * sb).cuda().T
    got = g.gemm(dev(a), dev(b), g.mx_tile_scales(dev(ea)), g.mx_tile_scales(dev(eb)), g.MX_TILED, c_dtype=g.FP32)
    assert torch.equal(got, want)
