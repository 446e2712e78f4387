"""a8w8_quantize on the GPU against the oracle's quantisers: bytes and scales bit for bit (integer /
byte work), for every scale mode, ragged shapes, padded rows, all-zero groups and extreme magnitudes."""
import numpy as np
import pytest
import torch

import gcnasm_amd as g
from gpu_util import dev

pytestmark = pytest.mark.gpu


def _x(rows, k, seed, wide=True):
    rng = np.random.Generator(np.random.Philox(seed))
    x = rng.standard_normal((rows, k)).astype(np.float32)
    if wide:
        x *= np.exp2(rng.integers(-30, 30, (rows, max(k // 32, 1)))).repeat(32, axis=1)[:, :k].astype(np.float32)
    x[rng.integers(0, rows), :] = 0            # an all-zero row
    return x


def _run(x, mode, group_rows=1):
    q, s = g.quantize(dev(x), mode, group_rows)
    torch.cuda.synchronize()
    return q.cpu().numpy(), s.cpu().numpy()


@pytest.mark.parametrize("rows,k", [(1, 32), (37, 96), (300, 1024), (2048, 4096)])
def test_per_tensor(orc, rows, k):
    x = _x(rows, k, 5 + rows, wide=False)
    q, s = _run(x, g.TENSOR)
    qr, sr = orc.quantize(x, orc.TENSOR)
    assert s.shape == (1,) and s.view(np.uint32)[0] == sr.view(np.uint32)[0]
    assert (q == qr).all()
    z = np.zeros((4, 64), np.float32)
    q, s = _run(z, g.TENSOR)
    assert s[0] == 1 and (q == 0).all()


@pytest.mark.parametrize("rows,k", [(1, 32), (37, 96), (256, 512), (130, 7168)])
def test_rowwise(orc, rows, k):
    x = _x(rows, k, 10 + rows)
    q, s = _run(x, g.ROWCOL)
    qr, sr = orc.quantize(x, orc.ROWCOL)
    assert (s.view(np.uint32) == sr.view(np.uint32)).all()
    assert (q == qr).all()


@pytest.mark.parametrize("rows,k", [(1, 128), (37, 384), (256, 2048)])
def test_block_1x128(orc, rows, k):
    x = _x(rows, k, 20 + rows)
    q, s = _run(x, g.BLOCK, 1)
    qr, sr = orc.quantize(x, orc.BLOCK, 1)
    assert s.shape == sr.shape and (s.view(np.uint32) == sr.view(np.uint32)).all()
    assert (q == qr).all()


@pytest.mark.parametrize("rows,k", [(128, 128), (384, 512)])
def test_block_128x128(orc, rows, k):
    x = _x(rows, k, 30 + rows)
    x[128:256, 0:128] = 0 if rows > 128 else x[128:256, 0:128]
    q, s = _run(x, g.BLOCK, 128)
    qr, sr = orc.quantize(x, orc.BLOCK, 128)
    assert s.shape == sr.shape and (s.view(np.uint32) == sr.view(np.uint32)).all()
    assert (q == qr).all()


@pytest.mark.parametrize("rows,k", [(1, 32), (37, 96), (256, 1024), (70, 7168)])
def test_mx(orc, rows, k):
    x = _x(rows, k, 40 + rows)
    x[0, :32] = [448 * 2.0 ** -3] + [0] * 31             # exactly a power of two times 448
    q, s = _run(x, g.MX)
    qr, sr = orc.quantize(x, orc.MX)
    assert (s == sr).all()
    assert (q == qr).all()


def test_extremes_and_padded_rows(orc):
    rows, k = 8, 256
    x = np.zeros((rows, k), np.float32)
    x[0, :4] = [3.0e38, -1.0e38, 1e-38, -1e-45]       # near fp32 max, a denormal
    x[1, :3] = [1e-40, 2e-40, -3e-41]                 # a row of denormals only
    x[2, :2] = [448.0, -447.9]
    x[3, 7] = -0.0
    for mode, gr in ((g.ROWCOL, 1), (g.BLOCK, 1), (g.MX, 1)):
        q, s = _run(x, mode, gr)
        qr, sr = orc.quantize(x, mode, gr)
        assert (q == qr).all(), mode
        assert (s.view(np.uint8) == sr.view(np.uint8)).all(), mode
    # a view with a row stride larger than k
    wide = _x(16, 512, 77)
    xv = dev(wide)[:, :256]
    q, s = g.quantize(xv, g.ROWCOL)
    qr, sr = orc.quantize(np.ascontiguousarray(wide[:, :256]), orc.ROWCOL)
    assert (q.cpu().numpy() == qr).all() and (s.cpu().numpy() == sr).all()


def test_quantize_then_gemm_matches_oracle_pipeline(orc):
    """The bytes and scales a8w8_quantize writes feed a8w8_gemm directly, in every mode."""
    m, n, k = 256, 256, 512
    a, b = _x(m, k, 91, wide=False), _x(n, k, 92, wide=False)
    for mode, ga, gb in ((g.TENSOR, 1, 1), (g.ROWCOL, 1, 1), (g.BLOCK, 1, 128), (g.MX, 1, 1), (g.MX_TILED, 1, 1)):
        qa, sa = g.quantize(dev(a), mode, ga)
        qb, sb = g.quantize(dev(b), mode, gb)
        c = g.gemm(qa, qb, sa, sb, mode, c_dtype=g.FP32).cpu().numpy()
        omode = orc.MX if mode == g.MX_TILED else mode
        oa, osa = orc.quantize(a, omode, ga)
        ob, osb = orc.quantize(b, omode, gb)
        ref = orc.gemm_ref(oa, ob, osa, osb, omode)
        assert (np.abs(c - ref) <= 1e-2 * np.abs(ref) + 1e-2).all(), mode


def test_vector_and_scalar_kernels_agree_with_the_oracle_on_views(orc):
    """16-byte aligned rows take the vectorised kernels (four or eight elements per thread), anything
    else the one-element-per-thread kernels: an aligned view with padded rows, a view that starts four
    bytes into its rows, and a row longer than a workgroup holds in registers."""
    rows, k = 70, 512
    big = _x(rows, 2 * k + 32, 123)
    views = {"padded rows": (slice(None), slice(0, k)), "offset by one element": (slice(None), slice(1, 1 + k))}
    for name, (r, c) in views.items():
        want = np.ascontiguousarray(big[r, c])
        xv = dev(big)[r, c]
        assert (xv.data_ptr() % 16 == 0) == (name == "padded rows")
        for mode, gr in ((g.TENSOR, 1), (g.ROWCOL, 1), (g.BLOCK, 1), (g.MX, 1), (g.MX_TILED, 1)):
            q, s = g.quantize(xv, mode, gr)
            qr, sr = orc.quantize(want, orc.MX if mode == g.MX_TILED else mode, gr)
            assert (q.cpu().numpy() == qr).all(), (name, mode)
            if mode == g.MX_TILED:
                assert (s.cpu().numpy() == orc.mx_tile_scales(sr)).all(), (name, mode)
            else:
                assert (s.cpu().numpy().view(np.uint8) == sr.view(np.uint8)).all(), (name, mode)
        q4, s4 = g.quantize_mxfp4(xv)
        qr4, sr4 = orc.quantize_mxfp4(want)
        assert (q4.cpu().numpy() == qr4).all() and (s4.cpu().numpy() == sr4).all(), name
    long_rows = _x(5, 16384, 124)
    q, s = _run(long_rows, g.ROWCOL)
    qr, sr = orc.quantize(long_rows, orc.ROWCOL)
    assert (q == qr).all() and (s.view(np.uint32) == sr.view(np.uint32)).all()
