"""GPU parity of the skinny-M flatmm over pre-shuffled weights."""
import ctypes

import numpy as np
import pytest

import datagen
import gcnasm_amd as g
from gpu_util import assert_close, assert_fp32_accurate, exact64, run_flatmm

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [(16, 256, 512), (16, 1024, 7168), (5, 48, 192), (33, 128, 256), (16, 16, 64)])
def test_flatmm_rowcol(orc, shape):
    m, n, k = shape
    a, b, sa, sb = datagen.row_col(m, n, k, seed=800 + n)
    bs = g.preshuffle_b(b)
    want = orc.flatmm_ref(a, bs, sa, sb, n)
    assert (want == orc.gemm_ref(a, b, sa, sb, orc.ROWCOL)).all()
    assert_close(run_flatmm(a, bs, sa, sb, n), want, f"flatmm {shape}")
    assert_fp32_accurate(run_flatmm(a, bs, sa, sb, n, c_dtype=g.FP32), *exact64(orc, a, b, sa, sb, g.ROWCOL))


def test_flatmm_exact_integers(orc):
    m, n, k = 16, 512, 1024
    a, b = datagen.small_ints(m, n, k, seed=31)
    want = orc.decode(a).astype(np.int64) @ orc.decode(b).astype(np.int64).T
    got = run_flatmm(a, g.preshuffle_b(b), np.ones(m, np.float32), np.ones(n, np.float32), n, c_dtype=g.FP32)
    assert (got == want).all()
    got = run_flatmm(a, g.preshuffle_b(b), np.ones(1, np.float32), np.ones(1, np.float32), n, mode=g.TENSOR,
                     c_dtype=g.FP32)
    assert (got == want).all()


# ---------------------------------------------------------------- MXFP8: E8M0 scales in the tiled layout

def _flat_mx(a, b, ea, eb, c_dtype=g.FP32):
    import torch
    from gpu_util import dev
    bs = g.preshuffle_b_device(dev(b))
    c = g.flatmm(dev(a), bs, g.mx_tile_scales(dev(ea)), g.mx_tile_scales(dev(eb)), b.shape[0], scale_mode=g.MX_TILED, c_dtype=c_dtype)
    torch.cuda.synchronize()
    return c.float().cpu().numpy()


@pytest.mark.parametrize("shape", [(16, 256, 512), (16, 1024, 7168), (5, 48, 192), (33, 128, 256), (64, 2048, 1024), (1, 16, 64)])
def test_flatmm_mx_against_the_oracle(orc, shape):
    m, n, k = shape
    a, b, ea, eb = datagen.mx(m, n, k, seed=900 + n)
    want = orc.gemm_ref(a, b, ea, eb, orc.MX)
    exact, mag = exact64(orc, a, b, ea, eb, g.MX)
    assert_fp32_accurate(_flat_mx(a, b, ea, eb), exact, mag)
    assert_close(_flat_mx(a, b, ea, eb, g.BF16), want, f"flatmm mx {shape}", exact=exact, mag=mag)


@pytest.mark.parametrize("case", range(24))
def test_flatmm_mx_scale_bytes_reach_the_right_lane_and_step(orc, case):
    """Small integers with a distinct power of two per (row, 32-block): sums are exact in fp32, so any mix-up of
    row, block or K step changes the result."""
    r = np.random.default_rng(8100 + case)
    m = int(r.integers(1, 129))
    n = 16 * int(r.integers(1, 70))
    k = 64 * int(r.integers(1, 40))
    a, b = datagen.small_ints(m, n, k, seed=8200 + case)
    ea = r.integers(125, 130, (m, k // 32)).astype(np.uint8)
    eb = r.integers(125, 130, (n, k // 32)).astype(np.uint8)
    A = orc.decode(a).astype(np.float64) * np.repeat(np.exp2(ea.astype(np.float64) - 127), 32, axis=1)
    B = orc.decode(b).astype(np.float64) * np.repeat(np.exp2(eb.astype(np.float64) - 127), 32, axis=1)
    got = _flat_mx(a, b, ea, eb)
    bad = np.argwhere(got != (A @ B.T).astype(np.float32))
    assert bad.size == 0, f"{m}x{n}x{k}: {len(bad)} elements differ, first {bad[:4].tolist()}"


# ---------------------------------------------------------------- block scales (1x128 / 128x128), the reference's layout

@pytest.mark.parametrize("shape", [(16, 256, 512), (16, 1024, 7168), (5, 128, 128), (33, 384, 256), (64, 2048, 1024)])
def test_flatmm_block_scales(orc, shape):
    import torch
    from gpu_util import dev
    m, n, k = shape
    a, b, sfa, sfb = datagen.block_scaled(m, n, k, seed=950 + n)
    want = orc.gemm_ref(a, b, sfa, sfb, orc.BLOCK)
    bs = g.preshuffle_b_device(dev(b))
    for c_dtype in (g.FP32, g.BF16):
        c = g.flatmm(dev(a), bs, dev(sfa), dev(sfb), n, scale_mode=g.BLOCK, c_dtype=c_dtype)
        torch.cuda.synchronize()
        got = c.float().cpu().numpy()
        if c_dtype == g.FP32:
            assert_fp32_accurate(got, *exact64(orc, a, b, sfa, sfb, g.BLOCK))
        else:
            assert_close(got, want, f"flatmm block {shape}")
    # the reference's own inputs and check (host.cc:46-63, 207-210): every element within 1e-3 absolute
    a, b, sfa, sfb = datagen.reference_style(m, n, k)
    c = g.flatmm(dev(a), g.preshuffle_b_device(dev(b)), dev(sfa), dev(sfb), n, scale_mode=g.BLOCK, c_dtype=g.FP32)
    assert orc.count_abs_mismatch(orc.gemm_ref(a, b, sfa, sfb, orc.BLOCK), c.cpu().numpy(), 1e-3) == 0


@pytest.mark.parametrize("case", range(16))
def test_flatmm_block_scales_exact(orc, case):
    """Small integers, power-of-two scales distinct per (row, K group) and per (128-row block, K group)."""
    import torch
    from gpu_util import dev
    r = np.random.default_rng(8300 + case)
    m = int(r.integers(1, 129))
    n = 128 * int(r.integers(1, 9))
    k = 128 * int(r.integers(1, 20))
    a, b = datagen.small_ints(m, n, k, seed=8400 + case)
    sfa = np.exp2(r.integers(-2, 3, (k // 128, m))).astype(np.float32)
    sfb = np.exp2(r.integers(-2, 3, (n // 128, k // 128))).astype(np.float32)
    A = orc.decode(a).astype(np.float64) * np.repeat(sfa.T.astype(np.float64), 128, axis=1)
    B = orc.decode(b).astype(np.float64) * np.repeat(np.repeat(sfb.astype(np.float64), 128, axis=0), 128, axis=1)
    c = g.flatmm(dev(a), g.preshuffle_b_device(dev(b)), dev(sfa), dev(sfb), n, scale_mode=g.BLOCK, c_dtype=g.FP32)
    torch.cuda.synchronize()
    bad = np.argwhere(c.cpu().numpy() != (A @ B.T).astype(np.float32))
    assert bad.size == 0, f"{m}x{n}x{k}: {len(bad)} elements differ, first {bad[:4].tolist()}"


# ---------------------------------------------------------------- several row groups per workgroup (M > 16)

def _row_group_case(orc, mode, m, n, k, batch, seed, rowmajor=False):
    """Exact small-integer problem, batched so that the launch picks the variant wanted; power-of-two scales
    distinct per row / group, so that a row group, weight tile, K block or scale taken from the wrong place
    changes the result."""
    import torch
    from gpu_util import dev
    r = np.random.default_rng(seed)
    a = np.stack([datagen.small_ints(m, n, k, seed=seed + 7 * i)[0] for i in range(batch)])
    b = np.stack([datagen.small_ints(m, n, k, seed=seed + 7 * i)[1] for i in range(batch)])
    A = orc.decode(a).astype(np.float64)
    B = orc.decode(b).astype(np.float64)
    if mode == g.ROWCOL:
        sfa = np.exp2(r.integers(-3, 4, (batch, m))).astype(np.float32)
        sfb = np.exp2(r.integers(-3, 4, (batch, n))).astype(np.float32)
        A, B = A * sfa[:, :, None], B * sfb[:, :, None]
        da, db = dev(sfa), dev(sfb)
    elif mode == g.TENSOR:
        sfa = np.exp2(r.integers(-3, 4, batch)).astype(np.float32)
        sfb = np.exp2(r.integers(-3, 4, batch)).astype(np.float32)
        A = A * (sfa * sfb).astype(np.float64)[:, None, None]
        da, db = dev(sfa), dev(sfb)
    elif mode == g.BLOCK:
        sfa = np.exp2(r.integers(-2, 3, (batch, k // 128, m))).astype(np.float32)
        sfb = np.exp2(r.integers(-2, 3, (batch, n // 128, k // 128))).astype(np.float32)
        A = A * np.repeat(np.swapaxes(sfa, 1, 2).astype(np.float64), 128, axis=2)
        B = B * np.repeat(np.repeat(sfb.astype(np.float64), 128, axis=1), 128, axis=2)
        da, db = dev(sfa), dev(sfb)
    else:
        ea = r.integers(125, 130, (batch, m, k // 32)).astype(np.uint8)
        eb = r.integers(125, 130, (batch, n, k // 32)).astype(np.uint8)
        A = A * np.repeat(np.exp2(ea.astype(np.float64) - 127), 32, axis=2)
        B = B * np.repeat(np.exp2(eb.astype(np.float64) - 127), 32, axis=2)
        da = torch.stack([g.mx_tile_scales(dev(ea[i])) for i in range(batch)])
        db = torch.stack([g.mx_tile_scales(dev(eb[i])) for i in range(batch)])
    if rowmajor:                                            # a8w8_gemm on row-major weights takes the flat kernel too
        bs = dev(b)
        args, c = g.api._args_from_tensors(dev(a), bs, da, db, mode, None, g.FP32, 0)
        entry = g.lib().a8w8_gemm
    else:
        bs = torch.stack([g.preshuffle_b_device(dev(b[i])) for i in range(batch)])
        args, c = g.api._args_from_tensors(dev(a), bs, da, db, mode, None, g.FP32, 1, n=n)
        entry = g.lib().a8w8_flatmm
    assert (args.stride_sfa_batch, args.stride_sfb_batch) == (da[0].numel(), db[0].numel())      # scales of their own per entry
    assert g.kernel_name(args) == "flatmm_a8w8"
    assert entry(ctypes.byref(args), g.api._stream()) == 0
    torch.cuda.synchronize()
    want = np.einsum("bmk,bnk->bmn", A, B).astype(np.float32)
    bad = np.argwhere(c.cpu().numpy() != want)
    assert bad.size == 0, f"mode {mode} {batch}x{m}x{n}x{k}: {len(bad)} elements differ, first {bad[:4].tolist()}"


@pytest.mark.parametrize("m", [17, 32, 33, 47, 48, 49, 63, 64, 65, 80, 97, 128])
@pytest.mark.parametrize("mode", [g.ROWCOL, g.TENSOR, g.MX_TILED, g.BLOCK])
def test_row_groups_two_weight_tiles(orc, mode, m):
    """Few weight tiles: two per workgroup, 2 / 3 / 4 row groups; 9 tiles leave the last workgroup half empty."""
    n, k = (144, 320) if mode in (g.ROWCOL, g.TENSOR) else (256, 384)      # 320 = an odd number of 64-wide K blocks
    _row_group_case(orc, mode, m, n, k, 2, 8500 + m)


@pytest.mark.parametrize("m", [17, 32, 33, 48, 49, 64, 81, 96, 113, 128])
@pytest.mark.parametrize("mode", [g.ROWCOL, g.TENSOR, g.MX_TILED, g.BLOCK])
def test_row_groups_four_weight_tiles(orc, mode, m):
    """At least four weight tiles per compute unit over all batch entries: four per workgroup (two for MX and block
    scales past 48 rows); 18 or 24 tiles per entry are not a multiple of four or leave the id remap without its
    multiple of eight."""
    n, k = (288, 192) if mode in (g.ROWCOL, g.TENSOR) else (384, 256)
    batch = (1024 * 16 + n - 1) // n
    _row_group_case(orc, mode, m, n, k, batch, 8600 + m)


@pytest.mark.parametrize("m", [1, 16, 17, 48, 64, 65, 96, 128])
@pytest.mark.parametrize("mode", [g.ROWCOL, g.TENSOR, g.MX_TILED, g.BLOCK])
@pytest.mark.parametrize("many_tiles", [False, True])
def test_row_major_weights_on_the_flat_kernel(orc, mode, m, many_tiles):
    """a8w8_gemm with row-major B and at most 128 rows: the flat kernel stages the weight rows through LDS.  Two or
    four weight tiles per workgroup, every count of row groups, ragged tile counts, an odd number of K blocks."""
    n, k = (144, 320) if mode in (g.ROWCOL, g.TENSOR) else (384, 256)
    batch = (1024 * 16 + n - 1) // n if many_tiles else 2
    _row_group_case(orc, mode, m, n, k, batch, 8800 + m, rowmajor=True)
