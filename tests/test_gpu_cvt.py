"""GPU parity of the fp8 <-> fp32 conversion helpers: bit-exact against the oracle."""
import numpy as np
import pytest
import torch

import gcnasm_amd as g
from gpu_util import dev

pytestmark = pytest.mark.gpu


def _sweep():
    rng = np.random.Generator(np.random.Philox(9))
    bits = rng.integers(0, 2 ** 32, 1 << 20, dtype=np.uint64).astype(np.uint32)
    # exponents 2^-14 .. 2^9 so that most samples fall in the representable range
    bits = (bits & np.uint32(0x807FFFFF)) | ((np.uint32(113) + (bits >> 23) % np.uint32(24)) << np.uint32(23))
    x = bits.view(np.float32)
    grid = np.arange(-4096, 4097, dtype=np.float32) / 8.0          # every tie of the coarse binades
    return np.concatenate([x, grid, np.array([0.0, -0.0, 240, -240, 448, -448, -54], np.float32)])


@pytest.mark.parametrize("dialect", [0, 1])
def test_decode_all_codes(orc, dialect):
    codes = np.arange(256, dtype=np.uint8)
    got = g.cvt_e4m3_to_f32(dev(codes), dialect).cpu().numpy()
    want = orc.decode(codes, dialect)
    nan = np.isnan(want)
    assert (np.isnan(got) == nan).all()
    assert (got[~nan].view(np.uint32) == want[~nan].view(np.uint32)).all()
    if dialect == 1:
        assert got.view(np.uint32)[0x80] == orc.cast_from_f8_bits(0x80, True)


@pytest.mark.parametrize("dialect", [0, 1])
def test_cvt_fp8_clamp240_bit_exact(orc, dialect):
    x = _sweep()
    got = g.cvt_f32_to_e4m3(dev(x), dialect, clamp240=True).cpu().numpy()
    want = orc.encode(x, dialect, clamp240=True)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, [(x[i], hex(got[i]), hex(want[i])) for i in bad[:5]]
    # the reference's single test input (cvt_fp8/test.cpp:133)
    one = g.cvt_f32_to_e4m3(dev(np.array([-54.0], np.float32)), dialect, clamp240=True).cpu().numpy()
    assert one[0] == (0xE6 if dialect == 0 else 0xEE)


@pytest.mark.parametrize("dialect", [0, 1])
def test_pk_cvt_unclamped_bit_exact_in_range(orc, dialect):
    x = _sweep()
    fmax = 448.0 if dialect == 0 else 240.0
    x = x[np.abs(x) <= fmax]
    x = x[: x.size // 4 * 4]
    got = g.cvt_f32_to_e4m3(dev(x), dialect, clamp240=False).cpu().numpy()
    want = orc.encode(x, dialect)
    assert (got == want).all()
    # packed byte order on the reference's own sweep i - 128 (pk_cvt/test.cpp:441-443)
    s = (np.arange(256) - 128).astype(np.float32)
    got = g.cvt_f32_to_e4m3(dev(s), dialect, clamp240=False).cpu().numpy()
    words = got.view(np.uint32)
    for i in range(64):
        assert words[i] == orc.pk_cvt_fp8x4(s[4 * i:4 * i + 4], dialect)


def test_ragged_lengths(orc):
    for n in (1, 2, 3, 5, 255, 257):
        x = np.linspace(-100, 100, n).astype(np.float32)
        got = g.cvt_f32_to_e4m3(dev(x), 0, clamp240=True).cpu().numpy()
        assert (got == orc.encode(x, 0, clamp240=True)).all()
    assert g.lib().a8w8_cvt_f32_to_e4m3(None, None, 4, 0, 0, None) == -1


def test_device_preshuffle(orc):
    rng = np.random.Generator(np.random.Philox(12))
    b = rng.integers(0, 256, (96, 320)).astype(np.uint8)
    got = g.preshuffle_b_device(dev(b)).cpu().numpy()
    assert (got == orc.preshuffle_b(b)).all()
