"""Seeded sweeps over the shapes and row strides of the entry points beside the dense FP8 GEMM: the flat
(skinny-M) GEMMs over pre-shuffled weights, the bf16 GEMM, the MXFP4 GEMM and the quantisers.  GEMM
operands are small integers (E2M1 codes for MXFP4) with power-of-two scales, so the float64 product is
what every kernel must return bit for bit; the quantisers are compared with the oracle byte for byte."""
import os

import numpy as np
import pytest
import torch

import gcnasm_amd as g
import oracle

pytestmark = pytest.mark.gpu

CASES = int(os.environ.get("A8W8_RANDOM_CASES", "24"))       # more cases for a longer soak of the same sweeps


def _view(r, x, pads, fill):
    """x [rows, cols] as a view into a wider GPU buffer with `fill` in the padding columns."""
    pad = int(r.choice(pads))
    whole = torch.full((x.shape[0], x.shape[1] + pad), fill, dtype=x.dtype, device="cuda")
    whole[:, : x.shape[1]] = x.cuda()
    return whole[:, : x.shape[1]], whole


def _check(c_view, c_whole, want, what):
    torch.cuda.synchronize()
    ref = torch.from_numpy(want.astype(np.float32)).to(c_view.dtype).float().numpy()
    got = c_view.float().cpu().numpy()
    bad = np.argwhere(got != ref)
    assert bad.size == 0, f"{what}: {len(bad)} of {got.size} elements differ, first {bad[:4].tolist()}"
    n = c_view.shape[1]
    if c_whole.shape[1] > n:
        assert (c_whole[:, n:].float() == 7.0).all(), f"{what}: wrote past column n"


def _c(r, m, n):
    cdt = [torch.bfloat16, torch.float32][int(r.integers(0, 2))]
    return _view(r, torch.zeros((m, n), dtype=cdt), [0, 0, 8, 3], 7.0)


@pytest.mark.parametrize("case", range(CASES))
def test_flatmm_fp8(case):
    r = np.random.default_rng(7000 + case)
    m = int(r.integers(1, 129))
    n = 16 * int(r.integers(1, 80))
    k = 64 * int(r.integers(1, 40))
    mode = [g.ROWCOL, g.TENSOR][case % 2]
    a = r.integers(-4, 5, (m, k)).astype(np.float32)
    b = r.integers(-4, 5, (n, k)).astype(np.float32)
    sfa = np.exp2(r.integers(-3, 4, m if mode == g.ROWCOL else 1)).astype(np.float32)
    sfb = np.exp2(r.integers(-3, 4, n if mode == g.ROWCOL else 1)).astype(np.float32)
    want = (a.astype(np.float64) * sfa[:, None]) @ (b.astype(np.float64) * sfb[:, None]).T
    da, _ = _view(r, torch.from_numpy(oracle.encode(a)), [0, 16, 64], 0x7F)      # flat GEMMs need 16-byte aligned A rows
    qb = torch.from_numpy(oracle.encode(b)).cuda()
    bs = g.preshuffle_b_device(qb)
    assert (bs.cpu().numpy() == g.preshuffle_b(oracle.encode(b))).all()
    c_view, c_whole = _c(r, m, n)
    what = f"flatmm case {case}: mode {mode} {m}x{n}x{k} lda={da.stride(0)} c={c_view.dtype} ldc={c_view.stride(0)}"
    print(what, flush=True)
    g.flatmm(da, bs, torch.from_numpy(sfa).cuda(), torch.from_numpy(sfb).cuda(), n, scale_mode=mode, c=c_view)
    _check(c_view, c_whole, want, what)


def test_flat_gemms_reject_misaligned_rows():
    a = torch.zeros((16, 64 + 5), dtype=torch.uint8, device="cuda")[:, :64]
    bs = torch.zeros(16 * 64, dtype=torch.uint8, device="cuda")
    one = torch.ones(16, dtype=torch.float32, device="cuda")
    with pytest.raises(g.A8W8Error, match="aligned"):
        g.flatmm(a, bs, one, one, 16)
    a16 = torch.zeros((16, 64 + 3), dtype=torch.bfloat16, device="cuda")[:, :64]
    with pytest.raises(g.A8W8Error, match="aligned"):
        g.flatmm_a16w16(a16, torch.zeros(16 * 128, dtype=torch.uint8, device="cuda"), 16)


@pytest.mark.parametrize("case", range(CASES))
def test_bf16_gemm_and_flat(case):
    r = np.random.default_rng(7100 + case)
    flat = case % 3 == 0
    m = int(r.integers(1, 129)) if flat else int(r.choice([1, 17, 64, 200, 256, 300, 513]))
    n = 16 * int(r.integers(1, 40)) if flat else int(r.choice([1, 24, 64, 255, 256, 384, 520]))
    k = 32 * int(r.integers(1, 40)) if flat else int(r.choice([8, 40, 64, 128, 192, 256, 448, 512, 1024]))
    a = torch.from_numpy(r.integers(-8, 9, (m, k)).astype(np.float32)).to(torch.bfloat16)
    b = torch.from_numpy(r.integers(-8, 9, (n, k)).astype(np.float32)).to(torch.bfloat16)
    want = a.double().numpy() @ b.double().numpy().T
    da, _ = _view(r, a, [0, 8, 32] if flat else [0, 8, 32, 3], 1.0)
    c_view, c_whole = _c(r, m, n)
    what = f"bf16 case {case}: flat={flat} {m}x{n}x{k} lda={da.stride(0)} c={c_view.dtype} ldc={c_view.stride(0)}"
    print(what, flush=True)
    if flat:
        g.flatmm_a16w16(da, g.preshuffle_b_bf16_device(b.cuda()), n, c=c_view)
    elif n % 16 == 0 and k % 64 == 0 and k >= 128 and da.stride(0) % 8 == 0:
        g.gemm_a16w16(da, g.preshuffle_b_bf16_device(b.cuda()), c=c_view, n=n)      # the dense kernels on shuffled weights
    else:
        db, _ = _view(r, b, [0, 8, 64, 1], 1.0)
        g.gemm_a16w16(da, db, c=c_view)
    _check(c_view, c_whole, want, what)


@pytest.mark.parametrize("case", range(CASES))
def test_mxfp4_gemm(case):
    r = np.random.default_rng(7200 + case)
    m = int(r.choice([1, 16, 63, 100, 256, 300, 520]))
    n = int(r.choice([1, 8, 64, 129, 256, 272, 512]))
    tiled = case % 2 == 0
    k = int(r.choice([512, 768, 1024, 256, 128])) if tiled else int(r.choice([32, 96, 128, 256, 480, 512]))
    # every E2M1 value is a multiple of 0.5 of magnitude <= 6 and block scales are 2^-1..2^1: sums stay exact in fp32
    qa = r.integers(0, 256, (m, k // 2)).astype(np.uint8)
    qb = r.integers(0, 256, (n, k // 2)).astype(np.uint8)
    ea = r.integers(126, 129, (m, k // 32)).astype(np.uint8)
    eb = r.integers(126, 129, (n, k // 32)).astype(np.uint8)
    A = oracle.e2m1_decode_packed(qa).astype(np.float64) * np.repeat(np.exp2(ea.astype(np.float64) - 127), 32, axis=1)
    B = oracle.e2m1_decode_packed(qb).astype(np.float64) * np.repeat(np.exp2(eb.astype(np.float64) - 127), 32, axis=1)
    da, _ = _view(r, torch.from_numpy(qa), [0, 16, 8], 0)
    db, _ = _view(r, torch.from_numpy(qb), [0, 16, 8], 0)
    dea, deb = torch.from_numpy(ea).cuda(), torch.from_numpy(eb).cuda()
    c_view, c_whole = _c(r, m, n)
    what = f"mxfp4 case {case}: tiled={tiled} {m}x{n}x{k} lda={da.stride(0) * 2} ldb={db.stride(0) * 2} c={c_view.dtype} ldc={c_view.stride(0)}"
    print(what, flush=True)
    if tiled and n % 16 == 0 and k % 256 == 0 and da.stride(0) % 16 == 0 and case % 4 == 0:
        g.gemm_a4w4(da, g.preshuffle_b_device(torch.from_numpy(qb).cuda()), g.mx_tile_scales(dea), g.mx_tile_scales(deb), g.MX_TILED,
                    c=c_view, n=n)                                                     # shuffled weights
    elif tiled:
        g.gemm_a4w4(da, db, g.mx_tile_scales(dea), g.mx_tile_scales(deb), g.MX_TILED, c=c_view)
    else:
        g.gemm_a4w4(da, db, dea, deb, g.MX, c=c_view)
    _check(c_view, c_whole, A @ B.T, what)


@pytest.mark.parametrize("case", range(CASES))
def test_quantisers(case):
    r = np.random.default_rng(7300 + case)
    mode, group_rows = [(g.TENSOR, 1), (g.ROWCOL, 1), (g.BLOCK, 1), (g.BLOCK, 128), (g.MX, 1), (g.MX_TILED, 1), ("fp4", 1)][case % 7]
    rows = int(r.choice([1, 7, 64, 100, 128, 300, 1024]))
    k = 128 * int(r.integers(1, 20)) if mode in (g.BLOCK, g.MX_TILED) else 32 * int(r.integers(1, 70))
    if group_rows == 128:
        rows = 128 * int(r.integers(1, 4))
    x = r.standard_normal((rows, k)).astype(np.float32)
    if mode != g.TENSOR:
        x *= np.exp2(r.integers(-20, 20, (rows, k // 32))).repeat(32, axis=1).astype(np.float32)
    x[int(r.integers(0, rows)), : 32 * int(r.integers(1, k // 32 + 1))] = 0        # an all-zero stretch
    xv, _ = _view(r, torch.from_numpy(x), [0, 0, 4, 32, 1], 1e30)                   # padding must not leak into any amax
    what = f"quantiser case {case}: mode {mode}/{group_rows} {rows}x{k} ld={xv.stride(0)}"
    print(what, flush=True)
    if mode == "fp4":
        q, s = g.quantize_mxfp4(xv)
        qr, sr = oracle.quantize_mxfp4(x)
    elif mode == g.MX_TILED:
        q, s = g.quantize(xv, g.MX_TILED)
        qr, sr = oracle.quantize(x, oracle.MX)
        sr = oracle.mx_tile_scales(sr)
    else:
        q, s = g.quantize(xv, mode, group_rows)
        qr, sr = oracle.quantize(x, mode, group_rows)
    torch.cuda.synchronize()
    assert (q.cpu().numpy() == qr).all(), what
    assert (s.cpu().numpy().view(np.uint8).ravel() == np.ascontiguousarray(sr).view(np.uint8).ravel()).all(), what
