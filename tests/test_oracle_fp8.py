"""Pins the oracle's FP8 / E8M0 / bf16 helpers against evidence that does not come from
the oracle: ROCm hip_fp8.h fixtures, closed forms, brute force and known answers."""
import math
import os
import struct

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _f(bits):
    return struct.unpack("<f", struct.pack("<I", bits))[0]


def _bits(f):
    return struct.unpack("<I", struct.pack("<f", f))[0]


def _load(name):
    rows = []
    with open(os.path.join(GOLD, name)) as fh:
        for line in fh:
            if line.startswith("#"):
                continue
            rows.append([int(t, 16) for t in line.split()])
    return rows


def test_decode_tables_match_hip_fp8(orc):
    for code, ocp_bits, fnuz_bits in _load("hip_fp8_decode.txt"):
        for dialect, want in ((orc.OCP, ocp_bits), (orc.FNUZ, fnuz_bits)):
            got = float(orc.decode(np.array([code], np.uint8), dialect)[0])
            if math.isnan(_f(want)):
                assert math.isnan(got), (code, dialect)
            else:
                assert _bits(got) == want, (hex(code), dialect)


def test_ocp_decode_closed_form(orc):
    for code in range(256):
        s, e, m = code >> 7, (code >> 3) & 15, code & 7
        got = float(orc.decode(np.array([code], np.uint8))[0])
        if e == 15 and m == 7:
            assert math.isnan(got)
            continue
        want = (m / 8) * 2.0 ** -6 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7)
        assert got == (-want if s else want)
    assert float(orc.decode(np.array([0x7E], np.uint8))[0]) == 448.0


def test_fnuz_two_reference_formulations_agree(orc):
    """closed form (cvt_fp8/test.cpp:59-90) vs bit manipulation (pk_cvt/test.cpp:340-421)."""
    for code in range(256):
        a = float(orc.decode(np.array([code], np.uint8), orc.FNUZ)[0])
        b = orc.cast_from_f8_bits(code, True)
        if code == 0x80:
            assert math.isnan(a) and b == 0x7F800001
        else:
            assert _bits(a) == b, hex(code)
    assert float(orc.decode(np.array([0x7F], np.uint8), orc.FNUZ)[0]) == 240.0


def test_cast_from_f8_ieee_mode(orc):
    """negative_zero_nan = false: bias 7, 0x80 = -0, exponent 15 = Inf/NaN."""
    assert orc.cast_from_f8_bits(0x80, False) == 0x80000000
    assert orc.cast_from_f8_bits(0x78, False) == 0x7F800000
    assert orc.cast_from_f8_bits(0xF8, False) == 0xFF800000
    assert orc.cast_from_f8_bits(0x79, False) == 0x7F800001
    for code in range(1, 0x78):   # finite codes coincide with OCP E4M3
        assert orc.cast_from_f8_bits(code, False) == _bits(float(orc.decode(np.array([code], np.uint8))[0]))


def test_encode_matches_hip_fp8(orc):
    rows = _load("hip_fp8_encode.txt")
    x = np.array([r[0] for r in rows], np.uint32).view(np.float32)
    assert (orc.encode(x, orc.OCP) == np.array([r[1] for r in rows], np.uint8)).all()
    got = orc.encode(x, orc.FNUZ)
    want = np.array([r[2] for r in rows], np.uint8)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, [(hex(rows[i][0]), hex(got[i]), hex(want[i])) for i in bad[:5]]


@pytest.mark.parametrize("dialect", [0, 1])
def test_encode_is_nearest_even_by_brute_force(orc, dialect):
    codes = np.arange(256, dtype=np.uint8)
    vals = orc.decode(codes, dialect).astype(np.float64)
    finite = ~np.isnan(vals) & (codes < 0x80)          # non-negative finite codes
    pc, pv = codes[finite], vals[finite]
    order = np.argsort(pv)
    pc, pv = pc[order], pv[order]
    rng = np.random.Generator(np.random.Philox(3))
    x = np.concatenate([
        rng.uniform(0, pv[-1], 20000),
        np.exp2(rng.uniform(-12, 9, 20000)),
        (pv[:-1] + pv[1:]) / 2,                          # exact ties
        pv,
    ]).astype(np.float32)
    x = x[x <= pv[-1]]
    got = orc.encode(x, dialect)
    for xi, gi in zip(x.astype(np.float64), got):
        d = np.abs(pv - xi)
        best = np.nonzero(d == d.min())[0]
        if best.size == 2:                               # tie -> even mantissa
            want = pc[best[0]] if pc[best[0]] % 2 == 0 else pc[best[1]]
        else:
            want = pc[best[0]]
        assert gi == want, (xi, hex(gi), hex(want))
    # negatives mirror positives
    neg = orc.encode(-x, dialect)
    nz = got != 0
    assert (neg[nz] == (got[nz] | 0x80)).all()


def test_encode_identity_and_specials(orc):
    codes = np.arange(256, dtype=np.uint8)
    for dialect, nan_codes in ((orc.OCP, (0x7F, 0xFF)), (orc.FNUZ, (0x80,))):
        vals = orc.decode(codes, dialect)
        back = orc.encode(vals, dialect)
        for c in range(256):
            if c in nan_codes:
                assert back[c] in nan_codes
            else:
                assert back[c] == c, (dialect, hex(c))
    assert orc.lib().orc_e4m3_ocp_encode(-54.0) == 0xE6            # tie -54 -> -56
    assert float(orc.decode(np.array([0xE6], np.uint8))[0]) == -56.0
    assert orc.lib().orc_e4m3_ocp_encode(1000.0) == 0x7E           # saturate to 448
    assert orc.lib().orc_e4m3_ocp_encode(float("inf")) == 0x7F
    assert orc.lib().orc_e4m3_fnuz_encode(-1e-9) == 0x00           # FNUZ has no -0


def test_cvt_fp8_clamp240(orc):
    L = orc.lib()
    assert L.orc_cvt_fp8_clamp240(1000.0, orc.OCP) == L.orc_e4m3_ocp_encode(240.0) == 0x77
    assert L.orc_cvt_fp8_clamp240(-1000.0, orc.OCP) == 0xF7
    assert L.orc_cvt_fp8_clamp240(1000.0, orc.FNUZ) == 0x7F
    assert L.orc_cvt_fp8_clamp240(-54.0, orc.FNUZ) == 0xEE          # cvt_fp8/test.cpp:133 input
    assert L.orc_cvt_fp8_clamp240(-54.0, orc.OCP) == 0xE6
    x = np.linspace(-239, 239, 1001).astype(np.float32)
    assert (orc.encode(x, orc.OCP, clamp240=True) == orc.encode(x, orc.OCP)).all()


def test_hardware_convert_matches_the_gfx950_record(orc):
    """orc_e4m3_ocp_encode_hw / orc_cvt_fp8_clamp240 against what the instruction returned on a gfx950
    device for NaN, Inf and out-of-range inputs (tests/golden/gfx950_cvt_pk_fp8_specials.txt)."""
    rows = _load("gfx950_cvt_pk_fp8_specials.txt")
    x = np.array([r[0] for r in rows], np.uint32).view(np.float32)
    got = orc.convert(x, orc.OCP)
    bad = [(hex(r[0]), hex(g_), hex(r[1])) for r, g_ in zip(rows, got) if g_ != r[1]]
    assert not bad, bad
    got = orc.encode(x, orc.OCP, clamp240=True)
    bad = [(hex(r[0]), hex(g_), hex(r[2])) for r, g_ in zip(rows, got) if g_ != r[2]]
    assert not bad, bad


def test_hardware_convert_is_the_saturating_one_where_nothing_overflows(orc):
    """Non-saturating and saturating conversions differ only for NaN and for magnitudes that round
    beyond 448: everywhere else the hip_fp8.h fixture pins both."""
    rows = _load("hip_fp8_encode.txt")
    x = np.array([r[0] for r in rows], np.uint32).view(np.float32)
    want = np.array([r[1] for r in rows], np.uint8)
    got = orc.convert(x, orc.OCP)
    with np.errstate(invalid="ignore"):
        over = np.isnan(x) | (np.abs(x) > 464.0)
    assert (got[~over] == want[~over]).all()
    assert over.sum() > 10
    sign = (x.view(np.uint32) >> 31).astype(np.uint8) << 7
    assert (got[over & ~np.isnan(x)] == (sign | 0x7F)[over & ~np.isnan(x)]).all()     # overflow, Inf: the NaN code, signed
    assert (got[np.isnan(x)] == 0xFF).all()
    # FNUZ: the saturating conversion of __hip_fp8_e4m3_fnuz throughout
    assert (orc.convert(x, orc.FNUZ) == np.array([r[2] for r in rows], np.uint8)).all()


def test_pk_cvt_byte_order(orc):
    """bytes come out as [f8(s0), f8(s1), f8(s2), f8(s3)] (perm selector 0x05040100)."""
    for base in range(-128, 124, 4):   # the harness sweep i - pixels/2, pk_cvt/test.cpp:441-443
        s = np.arange(base, base + 4, dtype=np.float32)
        word = orc.pk_cvt_fp8x4(s, orc.FNUZ)
        want = orc.encode(s, orc.FNUZ)
        assert [(word >> (8 * i)) & 0xFF for i in range(4)] == list(want)
    # selector semantics spelled out: result byte i = src byte sel_i of the 8-byte pool {y:x}
    x, y = 0x0000BBAA, 0x0000DDCC
    pool = x | (y << 32)
    sel = 0x05040100
    perm = sum(((pool >> (8 * ((sel >> (8 * i)) & 0xFF))) & 0xFF) << (8 * i) for i in range(4))
    assert perm == 0xDDCCBBAA


def test_e8m0(orc):
    assert orc.e8m0_decode(127) == 1.0
    assert orc.e8m0_decode(128) == 2.0
    assert orc.e8m0_decode(0) == 2.0 ** -127
    assert orc.e8m0_decode(254) == 2.0 ** 127
    assert math.isnan(orc.e8m0_decode(255))


def test_bf16_rne(orc):
    cases = {0x3F800000: 0x3F80, 0x3F808000: 0x3F80, 0x3F818000: 0x3F82, 0x3F808001: 0x3F81,
             0x7F7FFFFF: 0x7F80, 0xBF808000: 0xBF80, 0x00000000: 0x0000}
    for inp, want in cases.items():
        assert orc.lib().orc_f32_to_bf16(_f(inp)) == want, hex(inp)
    import torch
    x = np.random.Generator(np.random.Philox(5)).standard_normal(20000).astype(np.float32) * 100
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert (orc.to_bf16_bits(x) == want).all()
