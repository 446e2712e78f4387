"""The oracle's MXFP4 pieces against the OCP MX definition: the sixteen E2M1 values, nearest-even
encoding, GEMM against float64 on the decoded operands, quantiser properties."""
import numpy as np


def test_e2m1_value_table(orc):
    want = [0, 0.5, 1, 1.5, 2, 3, 4, 6]
    L = orc.lib()
    for c in range(8):
        assert L.orc_e2m1_decode(c) == want[c] and L.orc_e2m1_decode(c | 8) == -want[c]
    assert np.signbit(np.float32(L.orc_e2m1_decode(8)))          # negative zero


def test_e2m1_encode_nearest_even_and_saturation(orc):
    L = orc.lib()
    vals = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6], np.float64)
    for x in np.concatenate([np.linspace(-8, 8, 3201), [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 1e30, -1e30]]):
        code = L.orc_e2m1_encode(float(x))
        got = L.orc_e2m1_decode(code)
        d = np.abs(vals - abs(x))
        assert abs(abs(got) - abs(x)) == d.min()
        if (d == d.min()).sum() == 2:                              # a tie: the code with mantissa bit 0 wins
            assert (code & 1) == 0
        if x != 0:
            assert (got < 0) == (x < 0) or got == 0
    assert L.orc_e2m1_decode(L.orc_e2m1_encode(0.25)) == 0         # tie between 0 and 0.5 -> 0
    assert L.orc_e2m1_decode(L.orc_e2m1_encode(2.5)) == 2          # tie between 2 and 3 -> 2 (mantissa 0)
    assert L.orc_e2m1_decode(L.orc_e2m1_encode(5.0)) == 4          # tie between 4 and 6 -> 4
    assert L.orc_e2m1_decode(L.orc_e2m1_encode(100.0)) == 6


def test_mxfp4_gemm_against_float64(orc):
    rng = np.random.Generator(np.random.Philox(4))
    m, n, k = 9, 7, 96
    a = rng.integers(0, 256, (m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    ea = rng.integers(120, 134, (m, k // 32), dtype=np.uint8)
    eb = rng.integers(120, 134, (n, k // 32), dtype=np.uint8)
    A = orc.e2m1_decode_packed(a).astype(np.float64) * np.exp2(ea.astype(np.float64) - 127).repeat(32, axis=1)
    B = orc.e2m1_decode_packed(b).astype(np.float64) * np.exp2(eb.astype(np.float64) - 127).repeat(32, axis=1)
    got = orc.gemm_ref_mxfp4(a, b, ea, eb)
    assert np.abs(got - A @ B.T).max() <= 1e-5 * (np.abs(A) @ np.abs(B).T).max()
    # the low nibble is the even K index: a single non-zero element lands where it should
    a0 = np.zeros((1, 16), np.uint8); a0[0, 3] = 0x20                 # element 7 = code 2 = 1.0
    b0 = np.zeros((1, 16), np.uint8); b0[0, 3] = 0x70                 # element 7 = code 7 = 6.0
    e = np.full((1, 1), 127, np.uint8)
    assert orc.gemm_ref_mxfp4(a0, b0, e, e)[0, 0] == 6.0
    b0[0, 3] = 0x07                                                   # moved to element 6: no overlap
    assert orc.gemm_ref_mxfp4(a0, b0, e, e)[0, 0] == 0.0


def test_mxfp4_quantiser_properties(orc):
    rng = np.random.Generator(np.random.Philox(5))
    x = (rng.standard_normal((32, 256)) * np.exp2(rng.integers(-10, 10, (32, 8))).repeat(32, axis=1)).astype(np.float32)
    q, e = orc.quantize_mxfp4(x)
    d = orc.e2m1_decode_packed(q).reshape(32, 8, 32)
    top = np.abs(d).max(axis=2)
    assert (top <= 6).all() and (top >= 3).all()                     # tight, never saturating
    scale = np.exp2(e.astype(np.float64) - 127)[:, :, None]
    xs = x.reshape(32, 8, 32) / scale
    step = np.where(np.abs(xs) < 2, 0.5, np.where(np.abs(xs) < 4, 1.0, 2.0))
    assert (np.abs(d - xs) <= step / 2 + 1e-6).all()
    z, ez = orc.quantize_mxfp4(np.zeros((2, 64), np.float32))
    assert (z == 0).all() and (ez == 0).all()
