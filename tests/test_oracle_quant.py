"""The oracle's quantisers against what the recipe fixes (no reference code exists for them):
scale = amax/448, largest element -> +-448, error within half an E4M3 step, MX never saturates."""
import numpy as np
import pytest


def _x(rows, k, seed, spread=False):
    rng = np.random.Generator(np.random.Philox(seed))
    x = rng.standard_normal((rows, k)).astype(np.float32)
    if spread:
        x *= np.exp2(rng.integers(-20, 20, (rows, k // 32))).repeat(32, axis=1).astype(np.float32)
    return x


def _half_step(v):
    """Half the E4M3 spacing at |v| (3 mantissa bits, subnormal step 2^-9)."""
    a = np.maximum(np.abs(v), 2.0 ** -6)
    return np.exp2(np.floor(np.log2(a)) - 3) / 2


def test_rowwise_properties(orc):
    x = _x(37, 256, 1)
    q, s = orc.quantize(x, orc.ROWCOL)
    amax = np.abs(x).max(axis=1)
    assert (s == amax / np.float32(448)).all()
    d = orc.decode(q)
    assert (np.abs(d).max(axis=1) == 448).all()                      # the row's largest element hits the top code
    assert (np.abs(d - x / s[:, None]) <= _half_step(x / s[:, None]) * 1.0001).all()
    assert (np.sign(d) * np.sign(x) >= 0).all()


def test_per_tensor_properties(orc):
    x = _x(37, 256, 11)
    q, s = orc.quantize(x, orc.TENSOR)
    assert s.shape == (1,) and s[0] == np.abs(x).max() / np.float32(448)
    d = orc.decode(q)
    assert np.abs(d).max() == 448
    assert (np.abs(d - x / s[0]) <= _half_step(x / s[0]) * 1.0001).all()
    qr, sr = orc.quantize(x[:1], orc.ROWCOL)
    qt, st = orc.quantize(x[:1], orc.TENSOR)                 # one row: both recipes coincide
    assert (qr == qt).all() and sr[0] == st[0]


def test_block_properties_and_layouts(orc):
    x = _x(256, 384, 2)
    q1, s1 = orc.quantize(x, orc.BLOCK, 1)
    assert s1.shape == (3, 256)
    for g in range(3):
        assert (s1[g] == np.abs(x[:, g * 128:(g + 1) * 128]).max(axis=1) / np.float32(448)).all()
    q2, s2 = orc.quantize(x, orc.BLOCK, 128)
    assert s2.shape == (2, 3)
    for r in range(2):
        for g in range(3):
            blk = x[r * 128:(r + 1) * 128, g * 128:(g + 1) * 128]
            assert s2[r, g] == np.abs(blk).max() / np.float32(448)
            assert np.abs(orc.decode(q2[r * 128:(r + 1) * 128, g * 128:(g + 1) * 128])).max() == 448
    # both quantisers dequantise back to x within half a step of the scaled value
    d1 = orc.decode(q1) * s1.T.repeat(128, axis=1)
    assert np.abs(d1 - x).max() <= np.abs(x).max() * 2.0 ** -4


def test_mx_never_saturates_and_is_tight(orc):
    x = _x(64, 512, 3, spread=True)
    q, e = orc.quantize(x, orc.MX)
    d = orc.decode(q).reshape(64, 16, 32)
    top = np.abs(d).max(axis=2)
    assert (top <= 448).all() and (top > 224 * (1 - 2.0 ** -4)).all()
    scale = np.exp2(e.astype(np.float64) - 127)
    back = d * scale[:, :, None]
    xr = x.reshape(64, 16, 32)
    assert (np.abs(back - xr) <= _half_step(xr / scale[:, :, None]) * scale[:, :, None] * 1.0001).all()
    # an exact power of two times 448 needs no rounding up of the exponent
    y = np.zeros((1, 32), np.float32)
    y[0, 5] = 448 * 2.0 ** -3
    q, e = orc.quantize(y, orc.MX)
    assert e[0, 0] == 127 - 3 and orc.decode(q)[0, 5] == 448
    y[0, 5] = np.nextafter(np.float32(448 * 2.0 ** -3), np.float32(1e9))
    q, e = orc.quantize(y, orc.MX)
    assert e[0, 0] == 127 - 2


def test_all_zero_groups_stay_zero(orc):
    x = np.zeros((128, 256), np.float32)
    for mode, gr in ((orc.TENSOR, 1), (orc.ROWCOL, 1), (orc.BLOCK, 1), (orc.BLOCK, 128), (orc.MX, 1)):
        q, s = orc.quantize(x, mode, gr)
        assert (q == 0).all()
        assert (s == (0 if mode == orc.MX else 1)).all()


def test_quantised_gemm_tracks_the_fp32_product(orc):
    """End to end: quantise, run the oracle GEMM on bytes + scales, compare with the fp32 matmul."""
    a, b = _x(64, 256, 4), _x(128, 256, 5)
    want = a.astype(np.float64) @ b.astype(np.float64).T
    for mode, ga, gb in ((orc.TENSOR, 1, 1), (orc.ROWCOL, 1, 1), (orc.BLOCK, 1, 128), (orc.MX, 1, 1)):
        qa, sa = orc.quantize(a, mode, ga)
        qb, sb = orc.quantize(b, mode, gb)
        got = orc.gemm_ref(qa, qb, sa, sb, mode)
        err = np.abs(got - want).max() / np.abs(want).max()
        assert err < 0.05, (mode, err)
