"""Weight files (host only): what is saved comes back byte for byte, and a damaged, truncated or
foreign file is refused with the documented status."""
import ctypes
import os

import numpy as np
import pytest

import gcnasm_amd as g


def _weights(n, k, seed):
    rng = np.random.Generator(np.random.Philox(seed))
    return rng.integers(0, 256, (n, k), dtype=np.uint8)


@pytest.mark.parametrize("mode,n,k", [(g.TENSOR, 48, 192), (g.ROWCOL, 48, 192), (g.BLOCK, 256, 384), (g.MX, 48, 192),
                                      (g.MX_TILED, 70, 384)])
def test_round_trip(tmp_path, mode, n, k):
    b = _weights(n, k, 3 + mode)
    nbytes = g.lib().a8w8_weight_scale_bytes(n, k, mode)
    assert nbytes == {g.TENSOR: 4, g.ROWCOL: 4 * n, g.BLOCK: 4 * (n // 128) * (k // 128), g.MX: n * k // 32,
                      g.MX_TILED: g.mx_tiled_bytes(n, k)}[mode]
    rng = np.random.Generator(np.random.Philox(17))
    scales = rng.integers(0, 256, nbytes, dtype=np.uint8)
    scales = scales if mode in (g.MX, g.MX_TILED) else (scales.view(np.float32) if nbytes % 4 == 0 else scales)
    path = str(tmp_path / "w.a8w8")
    g.save_weights(path, b, scales, n, k, mode)
    assert os.path.getsize(path) == 64 + n * k + nbytes
    h, b2, s2 = g.load_weights(path)
    assert (h.n, h.k, h.scale_mode, h.b_preshuffled, h.version) == (n, k, mode, 0, 1)
    assert (b2 == b).all() and s2.tobytes() == scales.tobytes()


def test_preshuffled_weights_round_trip(tmp_path, orc):
    n, k = 64, 256
    b = _weights(n, k, 9)
    bs = g.preshuffle_b(b)
    path = str(tmp_path / "ws.a8w8")
    g.save_weights(path, bs, np.ones(n, np.float32), n, k, g.ROWCOL, b_preshuffled=True)
    h, b2, s2 = g.load_weights(path)
    assert h.b_preshuffled == 1 and (g.unshuffle_b(b2, n, k) == b).all() and (s2 == 1).all()


def test_damaged_files_are_refused(tmp_path):
    n, k = 32, 64
    path = str(tmp_path / "w.a8w8")
    g.save_weights(path, _weights(n, k, 1), np.ones(n, np.float32), n, k, g.ROWCOL)
    good = open(path, "rb").read()
    L = g.lib()
    buf_b, buf_s = np.empty(n * k, np.uint8), np.empty(4 * n, np.uint8)

    def load(data, cap_b=n * k, cap_s=4 * n):
        p2 = str(tmp_path / "x.a8w8")
        open(p2, "wb").write(data)
        return L.a8w8_weights_load(os.fsencode(p2), buf_b.ctypes.data, cap_b, buf_s.ctypes.data, cap_s)

    assert load(good) == 0
    flipped = bytearray(good); flipped[64 + 5] ^= 1
    assert load(bytes(flipped)) == -11                      # checksum
    assert load(good[:-3]) == -11                           # truncated payload
    assert load(good[:40]) == -11                           # truncated header
    assert load(b"NOTA8W8X" + good[8:]) == -11              # magic
    v2 = bytearray(good); v2[8] = 2
    assert load(bytes(v2)) == -11                           # version
    assert load(good, cap_b=n * k - 1) == -4                # caller's buffer too small
    assert L.a8w8_weights_load(os.fsencode(str(tmp_path / "missing")), buf_b.ctypes.data, n * k, buf_s.ctypes.data, 4 * n) == -10
    assert L.a8w8_weights_save(os.fsencode(str(tmp_path / "nodir" / "w")), buf_b.ctypes.data, buf_s.ctypes.data, n, k, 0, g.ROWCOL) == -10
    assert L.a8w8_weights_save(os.fsencode(path), buf_b.ctypes.data, buf_s.ctypes.data, n, 100, 0, g.BLOCK) == -3
    assert L.a8w8_weights_save(os.fsencode(path), buf_b.ctypes.data, buf_s.ctypes.data, n, k, 0, 9) == -6
    assert L.a8w8_weights_save(os.fsencode(path), None, buf_s.ctypes.data, n, k, 0, g.ROWCOL) == -1
    assert "checksum" in g.status_string(-11) and g.status_string(-10) != "unknown status"
