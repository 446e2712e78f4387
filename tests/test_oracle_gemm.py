"""Pins the oracle's GEMM / pre-shuffle restatements: float64 brute force on tiny shapes,
exact-integer inputs, reductions between scale modes, and permutation properties."""
import numpy as np
import pytest

import datagen


def _brute(orc, a, b, scale_fn):
    """float64 dense evaluation: sum_k A[i,k]*B[j,k]*scale(i,j,k) with numpy broadcasting."""
    A = orc.decode(a).astype(np.float64)
    B = orc.decode(b).astype(np.float64)
    m, k = A.shape
    n = B.shape[0]
    i, j, p = np.meshgrid(np.arange(m), np.arange(n), np.arange(k), indexing="ij")
    return (A[i, p] * B[j, p] * scale_fn(i, j, p)).sum(axis=2)


def test_block_scale_vs_brute_force(orc):
    m, n, k = 8, 256, 384
    a, b, sfa, sfb = datagen.block_scaled(m, n, k, seed=21)
    want = _brute(orc, a, b, lambda i, j, p: sfa[p // 128, i].astype(np.float64) * sfb[j // 128, p // 128])
    got = orc.gemm_ref(a, b, sfa, sfb, orc.BLOCK)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-4)
    # a transposed or mis-strided scale tensor must be visible at this tolerance
    bad = orc.gemm_ref(a, b, sfa[::-1].copy(), sfb, orc.BLOCK)
    assert not np.allclose(bad, want, rtol=2e-5, atol=2e-4)
    bad = orc.gemm_ref(a, b, sfa, sfb[:, ::-1].copy(), orc.BLOCK)
    assert not np.allclose(bad, want, rtol=2e-5, atol=2e-4)


def test_rowcol_and_tensor_vs_brute_force(orc):
    m, n, k = 9, 17, 96
    a, b, sa, sb = datagen.row_col(m, n, k, seed=22)
    want = _brute(orc, a, b, lambda i, j, p: sa[i].astype(np.float64) * sb[j])
    np.testing.assert_allclose(orc.gemm_ref(a, b, sa, sb, orc.ROWCOL), want, rtol=2e-5, atol=2e-4)
    a, b, sa, sb = datagen.per_tensor(m, n, k, seed=23)
    want = _brute(orc, a, b, lambda i, j, p: float(sa[0]) * float(sb[0]))
    np.testing.assert_allclose(orc.gemm_ref(a, b, sa, sb, orc.TENSOR), want, rtol=2e-5, atol=2e-4)


def test_mx_vs_brute_force(orc):
    m, n, k = 5, 12, 128
    a, b, ea, eb = datagen.mx(m, n, k, seed=24)
    assert ea.shape == (m, k // 32) and len(np.unique(ea)) > 2
    want = _brute(orc, a, b, lambda i, j, p: np.exp2(ea[i, p // 32].astype(np.float64) - 127)
                  * np.exp2(eb[j, p // 32].astype(np.float64) - 127))
    got = orc.gemm_ref(a, b, ea, eb, orc.MX)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-3 * np.abs(want).max() * 1e-2)
    # swapping the two scale tensors' block order must change the result
    bad = orc.gemm_ref(a, b, ea[:, ::-1].copy(), eb, orc.MX)
    assert not np.allclose(bad, want, rtol=1e-4)


def test_exact_integer_inputs_are_bit_exact(orc):
    m, n, k = 16, 128, 256
    a, b = datagen.small_ints(m, n, k)
    want = orc.decode(a).astype(np.int64) @ orc.decode(b).astype(np.int64).T
    one = np.ones(1, np.float32)
    assert (orc.gemm_ref(a, b, one, one, orc.TENSOR) == want).all()
    assert (orc.gemm_ref(a, b, np.ones(m, np.float32), np.ones(n, np.float32), orc.ROWCOL) == want).all()
    assert (orc.gemm_ref(a, b, np.ones((k // 128, m), np.float32), np.ones((n // 128, k // 128), np.float32),
                         orc.BLOCK) == want).all()
    e127 = lambda r: np.full((r, k // 32), 127, np.uint8)
    assert (orc.gemm_ref(a, b, e127(m), e127(n), orc.MX) == want).all()
    # power-of-two scales stay exact: MX with exponents == ROWCOL with the same powers of two
    ea = np.repeat(np.arange(m, dtype=np.uint8)[:, None] % 5 + 125, k // 32, axis=1)
    eb = np.repeat(np.arange(n, dtype=np.uint8)[:, None] % 3 + 126, k // 32, axis=1)
    sa = np.exp2(ea[:, 0].astype(np.float32) - 127)
    sb = np.exp2(eb[:, 0].astype(np.float32) - 127)
    assert (orc.gemm_ref(a, b, ea, eb, orc.MX) == orc.gemm_ref(a, b, sa, sb, orc.ROWCOL)).all()
    assert (orc.gemm_ref(a, b, ea, eb, orc.MX) == want * sa[:, None] * sb[None, :]).all()


def test_constant_scales_make_modes_coincide(orc):
    m, n, k = 8, 128, 256
    a, b = datagen.small_ints(m, n, k, seed=9)
    sa, sb = np.float32(0.75), np.float32(1.5)      # products stay exact
    t = orc.gemm_ref(a, b, np.array([sa]), np.array([sb]), orc.TENSOR)
    r = orc.gemm_ref(a, b, np.full(m, sa), np.full(n, sb), orc.ROWCOL)
    g = orc.gemm_ref(a, b, np.full((k // 128, m), sa), np.full((n // 128, k // 128), sb), orc.BLOCK)
    assert (t == r).all() and (t == g).all()


def test_rows_slab_and_probes_agree_with_full(orc):
    m, n, k = 24, 128, 256
    a, b, sfa, sfb = datagen.block_scaled(m, n, k, seed=31)
    full = orc.gemm_ref(a, b, sfa, sfb, orc.BLOCK)
    assert (orc.gemm_ref(a, b, sfa, sfb, orc.BLOCK, rows=(8, 16)) == full[8:16]).all()
    assert (orc.gemm_ref(a, b, sfa, sfb, orc.BLOCK, decode_per_mac=True) == full).all()
    pi = np.array([0, 3, 23, 7], np.int32)
    pj = np.array([0, 127, 64, 5], np.int32)
    assert (orc.gemm_probe(a, b, sfa, sfb, orc.BLOCK, pi, pj) == full[pi, pj]).all()
    a, b, ea, eb = datagen.mx(m, n, k, seed=32)
    full = orc.gemm_ref(a, b, ea, eb, orc.MX)
    assert (orc.gemm_probe(a, b, ea, eb, orc.MX, pi, pj) == full[pi, pj]).all()


def test_preshuffle_is_a_bijection_and_flatmm_equals_gemm(orc):
    n, k = 64, 256
    rng = np.random.Generator(np.random.Philox(41))
    b = rng.integers(0, 256, (n, k)).astype(np.uint8)
    bs = orc.preshuffle_b(b)
    assert sorted(bs.tolist()) == sorted(b.ravel().tolist())
    idx = np.array([[orc.lib().orc_preshuffle_index(i, j, k) for j in range(k)] for i in range(n)])
    assert sorted(idx.ravel().tolist()) == list(range(n * k))
    assert (orc.unshuffle_b(bs, n, k) == b).all()
    # layout statement: tile (n/16, k/64) is 1 KiB; inside it lane = (k%64)/16*16 + n%16 holds 16 K-bytes
    t = bs.reshape(n // 16, k // 64, 4, 16, 16)
    assert (t[2, 3, 1, 5] == b[2 * 16 + 5, 3 * 64 + 16:3 * 64 + 32]).all()
    a, bq, sa, sb = datagen.row_col(16, n, k, seed=42)
    c1 = orc.flatmm_ref(a, orc.preshuffle_b(bq), sa, sb, n)
    c2 = orc.gemm_ref(a, bq, sa, sb, orc.ROWCOL)
    assert (c1 == c2).all()


def test_reference_validator(orc):
    ref = np.zeros(100, np.float32)
    out = ref.copy()
    out[3] = 2e-3
    out[7] = 5e-4
    assert orc.count_abs_mismatch(ref, out, 1e-3) == 1


@pytest.mark.parametrize("gen", ["per_tensor", "row_col", "block_scaled", "mx"])
def test_generators_are_seeded_and_use_full_range(orc, gen):
    f = getattr(datagen, gen)
    x = f(128, 128, 256)
    y = f(128, 128, 256)
    for u, v in zip(x, y):
        assert (u == v).all()
    q = orc.decode(x[0])
    assert np.isfinite(q).all()
    assert np.abs(q).max() >= (224 if gen == "mx" else 448)   # amax maps to the top of E4M3


def test_mx_tiled_layout_is_a_bijection_with_127_padding(orc):
    """Full 64-row blocks and whole 512-wide K groups: tiling permutes the bytes (distinct values in,
    the same multiset out, untile inverts it).  Ragged shapes: every byte no (row, block) owns is 127."""
    rows, k = 128, 1024
    sf = (np.arange(rows * (k // 32)) % 251).astype(np.uint8).reshape(rows, k // 32)
    t = orc.mx_tile_scales(sf)
    assert t.size == rows * (k // 32) == orc.mx_tiled_bytes(rows, k)
    assert (np.sort(t) == np.sort(sf.ravel())).all()
    assert (orc.mx_untile_scales(t, rows, k) == sf).all()
    rows, k = 70, 384
    sf = np.full((rows, k // 32), 5, np.uint8)
    t = orc.mx_tile_scales(sf)
    assert t.size == 2 * 1024 and (t == 5).sum() == rows * (k // 32) and (t == 127).sum() == t.size - rows * (k // 32)
    assert (orc.mx_untile_scales(t, rows, k) == sf).all()


def test_mx_tiled_layout_groups_what_one_lane_needs(orc):
    """The eight bytes of (block, pair, r16, g) are two dwords of [tile parity][step]: byte (jp, par, s)
    belongs to row 32 jp + 8 (r16/4) + 4 par + r16%4 of the block and to K block 8 pair + 4 s + g."""
    rows, k = 64, 512
    sf = np.zeros((rows, k // 32), np.uint8)
    row, kblk = 32 * 1 + 8 * 2 + 4 * 1 + 3, 8 * 1 + 4 * 0 + 2      # jp=1, r16=11, par=1; pair=1, s=0, g=2
    sf[row, kblk] = 200
    t = orc.mx_tile_scales(sf)
    pos = int(np.nonzero(t == 200)[0][0])
    assert pos == ((1 * 64 + 11 * 4 + 2) * 8) + 1 * 4 + 1 * 2 + 0


def test_bf16_gemm_oracle_against_float64_and_integers(orc):
    rng = np.random.Generator(np.random.Philox(77))
    a = rng.standard_normal((9, 40)).astype(np.float32)
    b = rng.standard_normal((7, 40)).astype(np.float32)
    ab, bb = orc.to_bf16_bits(a), orc.to_bf16_bits(b)
    af, bf = orc.bf16_bits_to_f32(ab).astype(np.float64), orc.bf16_bits_to_f32(bb).astype(np.float64)
    got = orc.gemm_bf16_ref(ab, bb)
    assert np.abs(got - af @ bf.T).max() <= 1e-5 * (np.abs(af) @ np.abs(bf).T).max()
    ai = rng.integers(-8, 9, (5, 64)).astype(np.float32)
    bi = rng.integers(-8, 9, (6, 64)).astype(np.float32)
    assert (orc.gemm_bf16_ref(orc.to_bf16_bits(ai), orc.to_bf16_bits(bi)) == ai @ bi.T).all()
    # a transposed B would not pass: the oracle indexes B as [N, K]
    assert got.shape == (9, 7)
