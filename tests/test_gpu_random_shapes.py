"""Seeded sweep over shapes, row strides, batch counts, scale modes and output types of the dense GEMM
entry points.  Operands are small integers and scales powers of two, so every partial sum is exact in
fp32 whatever the order of accumulation and each kernel behind the entry points (pipelined four- and
eight-wave, plain tiled, one-thread-per-element) must give the float64 matrix product bit for bit;
padding columns of A, B and C must stay untouched."""
import os

import numpy as np
import pytest
import torch

import gcnasm_amd as g
import oracle

pytestmark = pytest.mark.gpu

CASES = int(os.environ.get("A8W8_RANDOM_CASES", "48"))       # more cases for a longer soak of the same sweep


def _dims(r):
    m = int(r.choice([1, 16, 63, 64, 100, 255, 256, 257, 300, 511, 640, 777]))
    n = int(r.choice([1, 8, 17, 64, 128, 129, 256, 272, 400, 512, 648]))
    k = int(r.choice([32, 96, 128, 256, 384, 512, 640, 1024, 1152]))
    return m, n, k


def _pow2(r, shape, lo, hi):
    return np.exp2(r.integers(lo, hi + 1, shape)).astype(np.float32)


def _padded(r, x, pad_choices, fill):
    """x [.., rows, cols] inside a wider buffer: returns (view on the GPU, whole buffer)."""
    pad = int(r.choice(pad_choices))
    shape = x.shape[:-1] + (x.shape[-1] + pad,)
    whole = torch.full(shape, fill, dtype=x.dtype, device="cuda")
    view = whole[..., : x.shape[-1]]
    view.copy_(x)
    return view, whole


@pytest.mark.parametrize("shuffled", [False, True], ids=["row_major_b", "shuffled_b"])
@pytest.mark.parametrize("case", range(CASES))
def test_random_case(case, shuffled):
    """shuffled: the same sweep with B in the pre-shuffled layout of the flat GEMM (whole 16-row groups and 128-wide
    K steps, aligned rows of A), which a8w8_gemm reads directly."""
    r = np.random.default_rng(9000 + case)
    mode = [g.TENSOR, g.ROWCOL, g.BLOCK, g.MX, g.MX_TILED][case % 5]
    m, n, k = _dims(r)
    if shuffled:
        n, k = -(-n // 16) * 16, max(128, k // 128 * 128)
    if mode == g.BLOCK:
        n = max(128, n // 128 * 128)            # the reference's block-scale program needs N and K in whole blocks
        k = max(128, k // 128 * 128)
    if mode == g.MX_TILED:
        k = max(128, k // 128 * 128)            # the tiled scale layout covers whole 128-wide K steps
    # small problems run on 128 x 128 tiles; many batch entries of a small shape put the same ragged tiles on the 256 x 256 kernels
    batch = int(r.choice([1, 1, 2, 3, 70, 140])) if m <= 300 and n <= 300 else int(r.choice([1, 1, 2, 3]))
    c_dtype = [g.BF16, g.FP32][int(r.integers(0, 2))]
    _exact_case(r, f"case {case}", mode, batch, m, n, k, c_dtype, shuffled)


@pytest.mark.parametrize("shuffled", [False, True], ids=["row_major_b", "shuffled_b"])
@pytest.mark.parametrize("mode", [g.TENSOR, g.ROWCOL, g.BLOCK, g.MX, g.MX_TILED])
@pytest.mark.parametrize("m,n,k,batch", [(130, 320, 2048, 1), (256, 1152, 2176, 1), (200, 128, 2304, 3), (257, 2048, 2048, 1)])
def test_short_wide_problems_on_narrow_tiles(m, n, k, batch, mode, shuffled):
    """A few hundred rows, a long K loop and so few 128 x 128 tiles that half of the compute units would idle: the
    128-tile kernel takes 128 x 64 tiles and five or six LDS stages (step counts that are and are not multiples of
    the stage count; a ragged last tile column; three M tiles)."""
    r = np.random.default_rng(9900 + m + n + k + 7 * mode)
    if mode == g.BLOCK:
        n = max(128, n // 128 * 128)            # block scales need N in whole blocks
    args = g.raw_gemm_args(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, m, n, k, mode, batch=batch, b_preshuffled=int(shuffled))
    assert g.kernel_name(args) == "gemm_a8w8_tile128"
    for c_dtype in (g.BF16, g.FP32):
        _exact_case(r, "narrow tiles", mode, batch, m, n, k, c_dtype, shuffled)


@pytest.mark.parametrize("mode", [g.TENSOR, g.ROWCOL, g.BLOCK, g.MX, g.MX_TILED])
@pytest.mark.parametrize("ksteps", [1, 2, 3, 4, 5, 7, 8, 9])
@pytest.mark.parametrize("m,n", [(384, 256), (2176, 2048)], ids=["four_stages", "two_stages"])
def test_overlapped_steps_of_the_128_tile_kernel(m, n, ksteps, mode):
    """The 128-tile kernel reads a step's fragments one step ahead (four stages: up to one tile per compute unit) or in
    front of a second barrier (two stages: up to two), and refills the stage between the MFMAs: every step count from
    one to past twice the stage count, odd and even (the four-stage loop is unrolled by two), exact in every scale mode."""
    k = 128 * ksteps
    r = np.random.default_rng(4200 + m + 13 * ksteps + 7 * mode)
    args = g.raw_gemm_args(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, m, n, k, mode)
    assert g.kernel_name(args) == "gemm_a8w8_tile128"
    _exact_case(r, f"{ksteps} K steps", mode, 1, m, n, k, g.FP32 if ksteps % 2 else g.BF16, False)


def _exact_case(r, label, mode, batch, m, n, k, c_dtype, shuffled):
    a = r.integers(-4, 5, (batch, m, k)).astype(np.float32)
    b = r.integers(-4, 5, (batch, n, k)).astype(np.float32)
    qa, qb = oracle.encode(a), oracle.encode(b)
    A, B = a.astype(np.float64), b.astype(np.float64)
    if mode == g.TENSOR:
        sfa, sfb = _pow2(r, (batch, 1), -2, 2), _pow2(r, (batch, 1), -2, 2)
        sA, sB = sfa[:, :, None], sfb[:, :, None]
    elif mode == g.ROWCOL:
        sfa, sfb = _pow2(r, (batch, m), -3, 3), _pow2(r, (batch, n), -3, 3)
        sA, sB = sfa[:, :, None], sfb[:, :, None]
    elif mode == g.BLOCK:
        sfa, sfb = _pow2(r, (batch, k // 128, m), -2, 2), _pow2(r, (batch, n // 128, k // 128), -2, 2)
        sA = np.repeat(np.swapaxes(sfa, 1, 2), 128, axis=2)
        sB = np.repeat(np.repeat(sfb, 128, axis=1), 128, axis=2)
    else:
        ea = r.integers(125, 130, (batch, m, k // 32)).astype(np.uint8)
        eb = r.integers(125, 130, (batch, n, k // 32)).astype(np.uint8)
        sA = np.repeat(np.exp2(ea.astype(np.float64) - 127), 32, axis=2)
        sB = np.repeat(np.exp2(eb.astype(np.float64) - 127), 32, axis=2)
        sfa, sfb = ea, eb
    want = np.einsum("bmk,bnk->bmn", A * sA, B * sB)

    da, _ = _padded(r, torch.from_numpy(qa), [0, 0, 16, 48] if shuffled else [0, 0, 16, 48, 5], 0x7F)
    db, _ = _padded(r, torch.from_numpy(qb), [0, 0, 16, 128, 3], 0x7F)
    if shuffled:
        db = torch.stack([g.preshuffle_b_device(db[i].contiguous()) for i in range(batch)])
    cdt = torch.bfloat16 if c_dtype == g.BF16 else torch.float32
    c_view, c_whole = _padded(r, torch.zeros((batch, m, n), dtype=cdt), [0, 0, 8, 24, 1], 7.0)
    dsa, dsb = torch.from_numpy(sfa).cuda(), torch.from_numpy(sfb).cuda()
    if mode == g.MX_TILED:
        tiles = [g.mx_tile_scales_ab(dsa[i], dsb[i]) for i in range(batch)]
        dsa = torch.stack([t[0] for t in tiles])
        dsb = torch.stack([t[1] for t in tiles])
    what = f"{label}{' (shuffled B)' if shuffled else ''}: mode {mode} {batch}x{m}x{n}x{k} c={c_dtype} lda={da.stride(-2)} ldb={db.stride(-2)} ldc={c_view.stride(-2)}"
    print(what, flush=True)
    if batch == 1:
        g.gemm(da[0], db[0], dsa[0], dsb[0], mode, c=c_view[0], n=n if shuffled else None)
    else:
        g.gemm(da, db, dsa, dsb, mode, c=c_view, n=n if shuffled else None)
    torch.cuda.synchronize()
    got = c_view.float().cpu().numpy()
    ref = torch.from_numpy(want.astype(np.float32)).to(cdt).float().numpy()
    bad = np.argwhere(got != ref)
    assert bad.size == 0, f"{what}: {len(bad)} elements differ, first {bad[:4].tolist()}"
    if c_whole.shape[-1] > n:
        assert (c_whole[..., n:].float() == 7.0).all(), f"{what}: wrote past column n"
