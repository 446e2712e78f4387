"""GPU parity of the dense GEMM entry points against the CPU oracle (through the C ABI).
Tolerance for floating-point cases: |C - Cref| <= 1e-2*|Cref| + 1e-2; exact-integer cases
must match bit for bit."""
import numpy as np
import pytest

import datagen
import gcnasm_amd as g
from gpu_util import assert_close, assert_fp32_accurate, dev, exact64, run_gemm

pytestmark = pytest.mark.gpu


def _scales_one(orc, mode, m, n, k):
    if mode == orc.TENSOR:
        return np.ones(1, np.float32), np.ones(1, np.float32)
    if mode == orc.ROWCOL:
        return np.ones(m, np.float32), np.ones(n, np.float32)
    if mode == orc.BLOCK:
        return np.ones((k // 128, m), np.float32), np.ones((n // 128, k // 128), np.float32)
    return np.full((m, k // 32), 127, np.uint8), np.full((n, k // 32), 127, np.uint8)


@pytest.mark.parametrize("mode", [0, 1, 2, 3])
@pytest.mark.parametrize("shape", [(256, 256, 256), (512, 256, 384), (64, 128, 128)])
def test_exact_integer_inputs_bit_exact(orc, mode, shape):
    m, n, k = shape
    a, b = datagen.small_ints(m, n, k, seed=100 + mode)
    sfa, sfb = _scales_one(orc, mode, m, n, k)
    want = orc.decode(a).astype(np.int64) @ orc.decode(b).astype(np.int64).T
    got = run_gemm(a, b, sfa, sfb, mode, c_dtype=g.FP32)
    assert (got == want).all(), np.argwhere(got != want)[:4]


def test_config1_per_tensor_256(orc):
    a, b, sa, sb = datagen.per_tensor(256, 256, 256)
    want = orc.gemm_ref(a, b, sa, sb, orc.TENSOR)
    assert_close(run_gemm(a, b, sa, sb, g.TENSOR), want, "C1 bf16")
    assert_fp32_accurate(run_gemm(a, b, sa, sb, g.TENSOR, g.FP32), *exact64(orc, a, b, sa, sb, g.TENSOR))


@pytest.mark.parametrize("shape", [(512, 512, 512), (300, 260, 256), (256, 520, 128), (1, 256, 128)])
def test_rowcol(orc, shape):
    m, n, k = shape
    a, b, sa, sb = datagen.row_col(m, n, k, seed=200 + m)
    want = orc.gemm_ref(a, b, sa, sb, orc.ROWCOL)
    assert_close(run_gemm(a, b, sa, sb, g.ROWCOL), want, f"rowcol {shape}")
    assert_fp32_accurate(run_gemm(a, b, sa, sb, g.ROWCOL, g.FP32), *exact64(orc, a, b, sa, sb, g.ROWCOL))


@pytest.mark.parametrize("shape", [(256, 256, 256), (512, 384, 1024), (100, 128, 384)])
def test_block_scale(orc, shape):
    m, n, k = shape
    a, b, sfa, sfb = datagen.block_scaled(m, n, k, seed=300 + m)
    want = orc.gemm_ref(a, b, sfa, sfb, orc.BLOCK)
    assert_close(run_gemm(a, b, sfa, sfb, g.BLOCK), want, f"block {shape}")
    assert_fp32_accurate(run_gemm(a, b, sfa, sfb, g.BLOCK, g.FP32), *exact64(orc, a, b, sfa, sfb, g.BLOCK))


def test_block_scale_reference_style_inputs_and_validator(orc):
    """The reference harness's own check: A~U[0,1), B~U[-.5,.5), scales~U[.8,1.2), fp32 out,
    every element within 1e-3 absolute (host.cc:46-63, 207-210, 273)."""
    m, n, k = 256, 512, 256                         # the reference's default problem (host.cc:134-136)
    a, b, sfa, sfb = datagen.reference_style(m, n, k)
    want = orc.gemm_ref(a, b, sfa, sfb, orc.BLOCK)
    c = g.gemm_blockscale(dev(a), dev(b), dev(sfa), dev(sfb))
    got = c.cpu().numpy()
    assert orc.count_abs_mismatch(want, got, 1e-3) == 0


def test_block_scale_batched(orc):
    batch, m, n, k = 3, 256, 256, 256
    per = [datagen.block_scaled(m, n, k, seed=400 + i) for i in range(batch)]
    a = np.stack([p[0] for p in per])
    b = np.stack([p[1] for p in per])
    sfa = np.stack([p[2] for p in per])
    sfb = np.stack([p[3] for p in per])
    c = g.gemm_blockscale(dev(a), dev(b), dev(sfa), dev(sfb)).cpu().numpy()
    for i in range(batch):
        want = orc.gemm_ref(a[i], b[i], sfa[i], sfb[i], orc.BLOCK)
        assert_close(c[i], want)
        assert_fp32_accurate(c[i], *exact64(orc, a[i], b[i], sfa[i], sfb[i], g.BLOCK))


@pytest.mark.parametrize("shape", [(256, 256, 256), (512, 256, 1024), (130, 270, 384)])
def test_mx(orc, shape):
    m, n, k = shape
    a, b, ea, eb = datagen.mx(m, n, k, seed=500 + m)
    want = orc.gemm_ref(a, b, ea, eb, orc.MX)
    exact, mag = exact64(orc, a, b, ea, eb, g.MX)
    assert_close(run_gemm(a, b, ea, eb, g.MX), want, f"mx {shape}", exact=exact, mag=mag)
    assert_fp32_accurate(run_gemm(a, b, ea, eb, g.MX, g.FP32), exact, mag)


def test_mx_scale_lanes_are_not_mixed_up(orc):
    """Each (row, 32-block) gets a distinct power of two; a wrong lane/byte selection in the
    scaled MFMA would move a scale to another row or block and change the exact result."""
    m, n, k = 256, 256, 256
    a, b = datagen.small_ints(m, n, k, seed=77, lo=-2, hi=2)
    # 2^-2..2^1 and 2^-1..2^1: with |a|,|b| <= 2 every partial sum stays an exact fp32 value
    ea = (125 + (np.arange(m)[:, None] * 3 + np.arange(k // 32)[None, :]) % 4).astype(np.uint8)
    eb = (126 + (np.arange(n)[:, None] * 5 + np.arange(k // 32)[None, :] * 2) % 3).astype(np.uint8)
    want = orc.gemm_ref(a, b, ea, eb, orc.MX)
    got = run_gemm(a, b, ea, eb, g.MX, g.FP32)
    assert (got == want).all()


@pytest.mark.parametrize("mode", [0, 1, 3])
def test_general_kernel_for_odd_shapes(orc, mode):
    """k % 128 != 0 takes the general kernel, which follows the oracle's order of operations."""
    m, n, k = 37, 53, 96
    if mode == 0:
        a, b, sa, sb = datagen.per_tensor(m, n, k, seed=601)
    elif mode == 1:
        a, b, sa, sb = datagen.row_col(m, n, k, seed=602)
    else:
        a, b, sa, sb = datagen.mx(m, n, k, seed=603)
    want = orc.gemm_ref(a, b, sa, sb, mode)
    got = run_gemm(a, b, sa, sb, mode, g.FP32)
    assert (got == want).all()
    assert_close(run_gemm(a, b, sa, sb, mode), want)


def test_strided_views(orc):
    import torch
    m, n, k = 256, 256, 256
    a, b, sa, sb = datagen.row_col(m, n, k, seed=700)
    want = orc.gemm_ref(a, b, sa, sb, orc.ROWCOL)
    abig = torch.zeros((m, k + 64), dtype=torch.uint8, device="cuda")
    abig[:, :k] = dev(a)
    cbig = torch.full((m, n + 8), 7.0, dtype=torch.bfloat16, device="cuda")
    g.gemm(abig[:, :k], dev(b), dev(sa), dev(sb), g.ROWCOL, c=cbig[:, :n])
    torch.cuda.synchronize()
    assert_close(cbig[:, :n].float().cpu().numpy(), want)
    assert (cbig[:, n:].float().cpu().numpy() == 7.0).all()      # nothing written past n
