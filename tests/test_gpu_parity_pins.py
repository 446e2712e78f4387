"""GPU checks that pin what the parity statements rest on.

* How the FP8 matrix-core instruction accumulates: the tolerance exception the MXFP8 configuration needs
  (a few outputs that cancel to almost zero miss |C - Cref| <= 1e-2*|Cref| + 1e-2) is justified by the
  instruction's own accumulation error, so that error is measured here against float64 and bounded.
* Conversion of NaN, Inf and out-of-range inputs on the hardware, against the oracle's statement of it.
* Routing corners: row strides of 2^23 bytes and more, a single K step over many tiles, one weight matrix shared
  by a batch, explicit device set-up.
* The whole-tile C stores (buffer stores through a per-tile descriptor) of both pipelined kernels, bit for bit, in
  both output types, into a C whose rows are padded; the same for the 128-tile kernel, whose whole tiles leave
  through LDS.
"""
import ctypes

import numpy as np
import pytest
import torch

import datagen
import gcnasm_amd as g
from gpu_util import MFMA_ACC_ERR, assert_close, dev, exact64

pytestmark = pytest.mark.gpu


def _wide_range_codes(rng, shape):
    """Uniformly random E4M3 codes (every exponent equally likely: magnitudes from 2^-9 to 448), NaN codes replaced."""
    x = rng.integers(0, 256, shape).astype(np.uint8)
    x[(x & 0x7F) == 0x7F] = 0x3C
    return x


@pytest.mark.parametrize("k", [128, 8192])
def test_mfma_accumulation_error_is_bounded_and_not_sequential(orc, k):
    """One 16 x 16 output tile, per-tensor scales of 1, fp32 out: the K products of an output are summed by K/128
    instructions of 128 products each.  The result stays within MFMA_ACC_ERR * sum|a||b| of the float64 value (the
    bound the MXFP8 tolerance exception uses) -- and it is NOT the sequentially rounded fp32 sum the CPU reference
    computes: on wide-range operands the instruction's error is several times that of the reference, which is why
    cancelling outputs can differ from the reference by more than the absolute tolerance whatever the kernel does."""
    rng = np.random.Generator(np.random.Philox(7000 + k))
    a, b = _wide_range_codes(rng, (16, k)), _wide_range_codes(rng, (16, k))
    one = np.ones(1, np.float32)
    got = g.gemm(dev(a), dev(b), dev(one), dev(one), g.TENSOR, c_dtype=g.FP32).cpu().numpy().astype(np.float64)
    exact, mag = exact64(orc, a, b, one, one, g.TENSOR)
    err = np.abs(got - exact) / mag
    assert err.max() <= MFMA_ACC_ERR, err.max()
    ref = orc.gemm_ref(a, b, one, one, orc.TENSOR).astype(np.float64)
    ref_err = np.abs(ref - exact) / mag
    assert ref_err.max() <= 2e-6, ref_err.max()               # sequential fp32: K roundings of 2^-24 each at worst
    if k == 8192:
        assert err.max() >= 3 * ref_err.max(), (err.max(), ref_err.max())
    # operands whose products and partial sums are integers below 2^24 lose nothing
    ai, bi = datagen.small_ints(16, 16, k, seed=k, lo=-4, hi=4)
    want = orc.decode(ai).astype(np.float64) @ orc.decode(bi).astype(np.float64).T
    got = g.gemm(dev(ai), dev(bi), dev(one), dev(one), g.TENSOR, c_dtype=g.FP32).cpu().numpy()
    assert (got == want).all()


def test_mfma_accumulation_error_on_the_mx_configuration_inputs(orc):
    """The same bound on the MXFP8 configuration's own input distribution (values N(0,1) * 2^U(-4,4) per block, E8M0
    scales) through both pipelined kernels, fp32 out: every output within MFMA_ACC_ERR * sum|a||b|s of float64."""
    m, n, k = 2304, 4096, 512                     # 144 tiles of 256 x 256: past the 128-tile kernel's range
    a, b, ea, eb = datagen.mx(m, n, k, seed=7100)
    exact, mag = exact64(orc, a, b, ea, eb, g.MX)
    da, db, dea, deb = dev(a), dev(b), dev(ea), dev(eb)
    name = lambda mode: g.kernel_name(g.raw_gemm_args(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, m, n, k, mode, g.FP32))
    assert name(g.MX) == "gemm_a8w8_persist" and name(g.MX_TILED) == "gemm_a8w8_wide"
    c_rm = g.gemm(da, db, dea, deb, g.MX, c_dtype=g.FP32).cpu().numpy()
    ta, tb = g.mx_tile_scales_ab(dea, deb)
    c_t = g.gemm(da, db, ta, tb, g.MX_TILED, c_dtype=g.FP32).cpu().numpy()
    for c in (c_rm, c_t):
        err = np.abs(c.astype(np.float64) - exact) / mag
        assert err.max() <= MFMA_ACC_ERR, err.max()
    assert (c_rm == c_t).all()


@pytest.mark.parametrize("dialect", [0, 1])
def test_conversion_of_nan_inf_and_overflow(orc, dialect):
    """NaN, +-Inf and magnitudes beyond the format through both conversion paths.  OCP is the hardware instruction:
    not saturating, overflow and Inf give the NaN code; FNUZ saturates; the +-240 clamp lets NaN/Inf through."""
    bits = np.array([0x7F800000, 0xFF800000, 0x7FC00000, 0xFFC00000, 0x7F800001, 0xFF800001, 0x7FFFFFFF, 0x7F7FFFFF,
                     0xFF7FFFFF], np.uint32).view(np.float32)
    vals = np.array([1e9, -1e9, 449, -449, 448, -448, 464, -464, 465, -465, 480, -480, 241, -241, 240, -240, 248, 256,
                     1e30, -1e30, 1e-30, -1e-30, 0.0, -0.0, 1000.0], np.float32)
    rng = np.random.Generator(np.random.Philox(77))
    big = (rng.uniform(200, 1200, 4096) * rng.choice([-1.0, 1.0], 4096)).astype(np.float32)      # around and beyond the maximum
    x = np.concatenate([bits, vals, big])
    x = np.concatenate([x, np.zeros((-x.size) % 4, np.float32)])
    got = g.cvt_f32_to_e4m3(dev(x), dialect, clamp240=False).cpu().numpy()
    want = orc.convert(x, dialect)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, [(hex(int(x.view(np.uint32)[i])), hex(got[i]), hex(want[i])) for i in bad[:8]]
    got = g.cvt_f32_to_e4m3(dev(x), dialect, clamp240=True).cpu().numpy()
    want = orc.encode(x, dialect, clamp240=True)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, [(hex(int(x.view(np.uint32)[i])), hex(got[i]), hex(want[i])) for i in bad[:8]]
    if dialect == 0:
        # the recorded answers of the instruction, and the packed form on a word that mixes all cases
        word = g.cvt_f32_to_e4m3(dev(np.array([np.inf, -1e9, np.nan, 464.0], np.float32)), 0).cpu().numpy()
        assert list(word) == [0x7F, 0xFF, 0xFF, 0x7E]
        assert int(word.view(np.uint32)[0]) == orc.pk_cvt_fp8x4(np.array([np.inf, -1e9, np.nan, 464.0], np.float32), 0)


def test_full_sweep_unclamped_including_out_of_range(orc):
    """The unclamped convert on a sweep that is NOT filtered to the representable range."""
    rng = np.random.Generator(np.random.Philox(78))
    bits = rng.integers(0, 2 ** 32, 1 << 18, dtype=np.uint64).astype(np.uint32)      # every exponent, NaNs and Infs included
    x = bits.view(np.float32)
    for dialect in (0, 1):
        got = g.cvt_f32_to_e4m3(dev(x), dialect, clamp240=False).cpu().numpy()
        want = orc.convert(x, dialect)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, [(hex(int(bits[i])), hex(got[i]), hex(want[i])) for i in bad[:8]]


def test_weight_rows_a_large_stride_apart(orc):
    """B as a strided view whose rows are 2^23 bytes apart (row offsets need full 32-bit products)."""
    m, n, k, ldb = 300, 17, 256, 1 << 23
    a, b, sa, sb = datagen.row_col(m, n, k, seed=7200)
    store = torch.zeros((n - 1) * ldb + k, dtype=torch.uint8, device="cuda")
    view = torch.as_strided(store, (n, k), (ldb, 1))
    view.copy_(dev(b))
    ref = orc.gemm_ref(a, b, sa, sb, orc.ROWCOL)
    for c_dtype in (g.BF16, g.FP32):
        c = g.gemm(dev(a), view, dev(sa), dev(sb), g.ROWCOL, c_dtype=c_dtype).float().cpu().numpy()
        assert datagen.tolerance_ok(c, ref).all()
    # 17 rows of B are not a multiple of 16: the MFMA kernel it is (the flat kernel needs whole 16-row tiles)
    args = g.raw_gemm_args(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, m, n, k, g.ROWCOL, stride_b=ldb)
    assert g.kernel_name(args) == "gemm_a8w8_tile128"


@pytest.mark.parametrize("mode", [g.ROWCOL, g.BLOCK, g.MX])
def test_single_k_step_over_many_tiles(orc, mode):
    """k = 128 on a problem of more 128 x 128 tiles than the chip holds at once (several rounds of workgroups)."""
    m, n, k = 2100, 4224, 128
    gen = {g.ROWCOL: datagen.row_col, g.BLOCK: datagen.block_scaled, g.MX: datagen.mx}[mode]
    a, b, sa, sb = gen(m, n, k, seed=7300 + mode)
    args = g.raw_gemm_args(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, m, n, k, mode)
    assert g.kernel_name(args) == "gemm_a8w8_tile128"
    c = g.gemm(dev(a), dev(b), dev(sa), dev(sb), mode, c_dtype=g.FP32).cpu().numpy()
    ref = orc.gemm_ref(a, b, sa, sb, mode)
    if mode == g.MX:      # wide-range inputs: outputs that cancel to almost zero are judged against float64
        exact, mag = exact64(orc, a, b, sa, sb, mode)
        assert_close(c, ref, "single K step", exact=exact, mag=mag)
    else:
        assert datagen.tolerance_ok(c, ref).all()
    ai, bi = datagen.small_ints(m, n, k, seed=7310, lo=-3, hi=3)
    want = orc.decode(ai).astype(np.float32) @ orc.decode(bi).astype(np.float32).T
    got = g.gemm(dev(ai), dev(bi), dev(np.ones(m, np.float32)), dev(np.ones(n, np.float32)), g.ROWCOL, c_dtype=g.FP32).cpu().numpy()
    assert (got == want).all()


def test_batch_sharing_one_weight_matrix(orc):
    """a [batch, m, k] with a 2-D b: every batch entry multiplies the same weights (batch stride 0 for B and its scales)."""
    batch, m, n, k = 3, 130, 272, 256
    per = [datagen.row_col(m, n, k, seed=7400 + i) for i in range(batch)]
    a = np.stack([p[0] for p in per])
    sa = np.stack([p[2] for p in per])
    b, sb = per[0][1], per[0][3]
    c = g.gemm(dev(a), dev(b), dev(sa), dev(sb), g.ROWCOL, c_dtype=g.FP32).cpu().numpy()
    for i in range(batch):
        ref = orc.gemm_ref(a[i], b, sa[i], sb, orc.ROWCOL)
        assert datagen.tolerance_ok(c[i], ref).all(), i
    with pytest.raises(ValueError):
        g.gemm(dev(a), dev(np.stack([b, b])), dev(sa), dev(sb), g.ROWCOL)          # two weight matrices for three entries
    with pytest.raises(ValueError):
        g.gemm(dev(a)[:, :, ::2], dev(b)[:, ::2], dev(sa), dev(sb), g.ROWCOL)      # rows that are not contiguous
    with pytest.raises(TypeError):
        g.gemm(dev(a), dev(b), dev(sa.astype(np.float64)), dev(sb), g.ROWCOL)
    with pytest.raises(ValueError, match="per entry"):
        g.gemm(dev(a), dev(b), dev(sa), dev(np.stack([sb] * batch)), g.ROWCOL)       # a set of weight scales per entry for shared weights
    with pytest.raises(ValueError, match="sfa holds"):
        g.gemm(dev(a), dev(b), dev(sa[:2]), dev(sb), g.ROWCOL)                       # scales of two entries for three
    with pytest.raises(ValueError, match="sfb holds"):
        g.gemm(dev(a), dev(b), dev(sa), dev(sb[: n - 1]), g.ROWCOL)


def test_explicit_device_setup():
    L = g.lib()
    assert L.a8w8_init(-1) == 0 and L.a8w8_init(0) == 0
    assert L.a8w8_init(63) == -9                                # no such device
    assert torch.cuda.current_device() == 0
    g.init()


@pytest.mark.parametrize("k", [512, 384])       # an even number of K steps: the four-wave kernel; odd: the eight-wave one
@pytest.mark.parametrize("c_dtype", [g.BF16, g.FP32])
def test_whole_tile_stores_bit_for_bit(orc, k, c_dtype):
    """Exact integers with row/col scales that are powers of two: every output is exact in fp32 (bf16: its one
    rounding, to nearest even on both sides), so any byte a store drops, moves or overwrites shows.  C has padded rows (stride_c > n), must keep its padding, and is
    written by workgroups that run two tiles back to back (more tiles than compute units)."""
    m, n, ldc = 4352, 4608, 4608 + 64
    a, b = datagen.small_ints(m, n, k, seed=7300 + k, lo=-1, hi=1)
    rng = np.random.Generator(np.random.Philox(7301))
    sa = np.exp2(rng.integers(-2, 3, m)).astype(np.float32)
    sb = np.exp2(rng.integers(-2, 3, n)).astype(np.float32)
    want = (torch.from_numpy(orc.decode(a)).cuda() @ torch.from_numpy(orc.decode(b)).cuda().T) * dev(sa)[:, None] * dev(sb)[None, :]
    torch_dtype = torch.bfloat16 if c_dtype == g.BF16 else torch.float32
    store = torch.full((m, ldc), -7.0, dtype=torch_dtype, device="cuda")
    c = store[:, :n]
    g.gemm(dev(a), dev(b), dev(sa), dev(sb), g.ROWCOL, c=c, c_dtype=c_dtype)
    args = g.raw_gemm_args(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, m, n, k, g.ROWCOL, c_dtype=c_dtype, stride_c=ldc)
    assert g.kernel_name(args) == ("gemm_a8w8_wide" if k == 512 else "gemm_a8w8_persist")
    assert torch.equal(c.float(), want.to(torch_dtype).float())
    assert bool((store[:, n:] == -7.0).all())


@pytest.mark.parametrize("c_dtype", [g.BF16, g.FP32])
def test_whole_tile_stores_with_tiled_mx_scales(orc, c_dtype):
    """The four-wave kernel deals the rows of a tile to its lanes differently when the scales are tiled MX; the
    stores have to follow.  Exact integers, per-row exponents that differ from row to row (a row that lands in
    another row's place shows), padded C."""
    m, n, k, ldc = 4352, 4608, 512, 4608 + 32
    a, b = datagen.small_ints(m, n, k, seed=7400, lo=-1, hi=1)
    rng = np.random.Generator(np.random.Philox(7401))
    ea = np.repeat(rng.integers(125, 130, (m, 1)), k // 32, axis=1).astype(np.uint8)
    eb = np.repeat(rng.integers(125, 130, (n, 1)), k // 32, axis=1).astype(np.uint8)
    sa = np.exp2(ea[:, 0].astype(np.float32) - 127)
    sb = np.exp2(eb[:, 0].astype(np.float32) - 127)
    want = (torch.from_numpy(orc.decode(a)).cuda() @ torch.from_numpy(orc.decode(b)).cuda().T) * dev(sa)[:, None] * dev(sb)[None, :]
    torch_dtype = torch.bfloat16 if c_dtype == g.BF16 else torch.float32
    store = torch.full((m, ldc), -7.0, dtype=torch_dtype, device="cuda")
    c = store[:, :n]
    g.gemm(dev(a), dev(b), g.mx_tile_scales(dev(ea)), g.mx_tile_scales(dev(eb)), g.MX_TILED, c=c, c_dtype=c_dtype)
    assert torch.equal(c.float(), want.to(torch_dtype).float())
    assert bool((store[:, n:] == -7.0).all())


@pytest.mark.parametrize("k", [256, 384])
@pytest.mark.parametrize("c_dtype", [g.BF16, g.FP32])
def test_c_rows_millions_of_elements_apart(orc, k, c_dtype):
    """stride_c = 4,000,000: the byte offsets of a C tile's rows pass 2^31 (unsigned 32-bit offsets in the kernels);
    enough 128-tiles that the pipelined kernels take the problem."""
    m, n, ldc = 256, 128 * 257, 4_000_000
    a, b = datagen.small_ints(m, n, k, seed=7500 + k, lo=-1, hi=1)
    want = torch.from_numpy(orc.decode(a)).cuda() @ torch.from_numpy(orc.decode(b)).cuda().T
    torch_dtype = torch.bfloat16 if c_dtype == g.BF16 else torch.float32
    store = torch.empty(m * ldc, dtype=torch_dtype, device="cuda")
    c = torch.as_strided(store, (m, n), (ldc, 1))
    ones_m, ones_n = dev(np.ones(m, np.float32)), dev(np.ones(n, np.float32))
    g.gemm(dev(a), dev(b), ones_m, ones_n, g.ROWCOL, c=c, c_dtype=c_dtype)
    args = g.raw_gemm_args(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, m, n, k, g.ROWCOL, c_dtype=c_dtype, stride_c=ldc)
    assert g.kernel_name(args) == ("gemm_a8w8_wide" if k == 256 else "gemm_a8w8_persist")
    assert torch.equal(c.float(), want.to(torch_dtype).float())
    del store
    torch.cuda.empty_cache()


@pytest.mark.parametrize("shape", [(256, 384, 256), (384, 256, 2304), (256, 192, 384)], ids=["wide_tiles", "narrow_tiles", "ragged_last_column"])
@pytest.mark.parametrize("c_dtype", [g.BF16, g.FP32])
def test_small_kernel_whole_tile_stores_bit_for_bit(orc, shape, c_dtype):
    """The 128-tile kernel sends tiles that lie inside the matrix through LDS and stores them along the rows.  Exact
    integers with power-of-two row/col scales: any value that lands in the wrong row or column shows.  C has padded
    rows, which must keep their padding; the third shape ends with a tile column that is not whole (stored from the
    registers, element by element where it crosses the edge); the second takes 128 x 64 tiles."""
    m, n, k = shape
    ldc = n + 40
    a, b = datagen.small_ints(m, n, k, seed=7400 + n, lo=-2, hi=2)
    rng = np.random.Generator(np.random.Philox(7401))
    sa = np.exp2(rng.integers(-2, 3, m)).astype(np.float32)
    sb = np.exp2(rng.integers(-2, 3, n)).astype(np.float32)
    want = (torch.from_numpy(orc.decode(a)).cuda() @ torch.from_numpy(orc.decode(b)).cuda().T) * dev(sa)[:, None] * dev(sb)[None, :]
    torch_dtype = torch.bfloat16 if c_dtype == g.BF16 else torch.float32
    store = torch.full((m, ldc), -7.0, dtype=torch_dtype, device="cuda")
    c = store[:, :n]
    g.gemm(dev(a), dev(b), dev(sa), dev(sb), g.ROWCOL, c=c, c_dtype=c_dtype)
    args = g.raw_gemm_args(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, m, n, k, g.ROWCOL, c_dtype=c_dtype, stride_c=ldc)
    assert g.kernel_name(args) == "gemm_a8w8_tile128"
    assert torch.equal(c.float(), want.to(torch_dtype).float())
    assert bool((store[:, n:] == -7.0).all())
