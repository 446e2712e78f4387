"""The bf16 sibling (a16w16_gemm) against the oracle: exact on integer inputs and on the general kernel,
|C - Cref| <= 1e-2*|Cref| + 1e-2 for bf16 outputs, fp32 outputs within 1e-5 of sum|a||b|."""
import numpy as np
import pytest
import torch

import gcnasm_amd as g

pytestmark = pytest.mark.gpu


def _bits(x):
    return x.view(torch.int16).cpu().numpy().view(np.uint16)


def _rand(m, k, seed):
    gen = torch.Generator(device="cuda"); gen.manual_seed(seed)
    return torch.randn((m, k), generator=gen, device="cuda").to(torch.bfloat16)


# (the last two: short and wide with a long K loop, which the 128-tile kernel runs on 128 x 64 tiles)
@pytest.mark.parametrize("shape", [(256, 256, 128), (512, 384, 1024), (130, 270, 192), (64, 64, 4096), (300, 520, 64 * 7),
                                   (200, 1088, 1024), (256, 320, 1088)])
def test_pipelined_kernel(orc, shape):
    m, n, k = shape
    a, b = _rand(m, k, 1 + m), _rand(n, k, 2 + n)
    ref = orc.gemm_bf16_ref(_bits(a), _bits(b))
    c = g.gemm_a16w16(a, b).float().cpu().numpy()
    assert (np.abs(c - ref) <= 1e-2 * np.abs(ref) + 1e-2).all()
    c32 = g.gemm_a16w16(a, b, c_dtype=g.FP32).cpu().numpy()
    mag = np.abs(a.float().cpu().numpy()).astype(np.float64) @ np.abs(b.float().cpu().numpy()).astype(np.float64).T
    exact = a.double().cpu().numpy() @ b.double().cpu().numpy().T
    assert (np.abs(c32 - exact) <= 1e-5 * mag + 1e-30).all()


def test_exact_integers_every_tile_and_step(orc):
    m, n, k = 768, 1024, 512
    gen = torch.Generator(device="cuda"); gen.manual_seed(5)
    a = torch.randint(-8, 9, (m, k), generator=gen, device="cuda").to(torch.bfloat16)
    b = torch.randint(-8, 9, (n, k), generator=gen, device="cuda").to(torch.bfloat16)
    want = a.float() @ b.float().T
    assert torch.equal(g.gemm_a16w16(a, b, c_dtype=g.FP32), want)
    assert (orc.gemm_bf16_ref(_bits(a), _bits(b)) == want.cpu().numpy()).all()


@pytest.mark.parametrize("shape", [(37, 53, 96), (16, 16, 40), (70, 40, 64)])
def test_general_kernel_is_bit_exact(orc, shape):
    m, n, k = shape
    a, b = _rand(m, k, 11), _rand(n, k, 12)
    ref = orc.gemm_bf16_ref(_bits(a), _bits(b))
    assert (g.gemm_a16w16(a, b, c_dtype=g.FP32).cpu().numpy() == ref).all()


def test_batched_and_strided(orc):
    batch, m, n, k = 3, 260, 300, 256
    a = torch.stack([_rand(m, k, 20 + i) for i in range(batch)])
    b = torch.stack([_rand(n, k, 30 + i) for i in range(batch)])
    c = g.gemm_a16w16(a, b, c_dtype=g.FP32).cpu().numpy()
    for i in range(batch):
        ref = orc.gemm_bf16_ref(_bits(a[i]), _bits(b[i]))
        np.testing.assert_allclose(c[i], ref, rtol=1e-4, atol=1e-4 * np.abs(ref).max())
    wide = _rand(256, 1024, 40)
    av = wide[:, 256:768]                                   # a view: row stride 1024, offset 512 bytes
    bb = _rand(256, 512, 41)
    ref = orc.gemm_bf16_ref(_bits(av.contiguous()), _bits(bb))
    np.testing.assert_allclose(g.gemm_a16w16(av, bb, c_dtype=g.FP32).cpu().numpy(), ref, rtol=1e-4, atol=1e-4 * np.abs(ref).max())


def test_full_size_4096(orc):
    m = n = k = 4096
    a, b = _rand(m, k, 50), _rand(n, k, 51)
    c = g.gemm_a16w16(a, b).float()
    ref = orc.gemm_bf16_ref(_bits(a[:16]), _bits(b))
    got = c[:16].cpu().numpy()
    assert (np.abs(got - ref) <= 1e-2 * np.abs(ref) + 1e-2).all()
    # doubling A doubles C exactly; permuting A's rows permutes C's rows bit for bit
    assert torch.equal(g.gemm_a16w16(a * 2, b).float(), 2 * c)
    perm = torch.randperm(m, generator=torch.Generator().manual_seed(3)).cuda()
    assert torch.equal(g.gemm_a16w16(a[perm].contiguous(), b), g.gemm_a16w16(a, b)[perm])


@pytest.mark.parametrize("shape", [(16, 256, 512), (1, 64, 32), (33, 2048, 1024), (64, 128, 96)])
def test_flat_gemm_over_preshuffled_bf16_weights(orc, shape):
    m, n, k = shape
    a, b = _rand(m, k, 61 + m), _rand(n, k, 62 + n)
    bs = g.preshuffle_b_bf16_device(b)
    # the device shuffle of the byte view is the oracle's shuffle of the same bytes
    assert (bs.cpu().numpy() == orc.preshuffle_b(b.view(torch.uint8).view(n, 2 * k).cpu().numpy())).all()
    ref = orc.gemm_bf16_ref(_bits(a), _bits(b))
    c32 = g.flatmm_a16w16(a, bs, n, c_dtype=g.FP32).cpu().numpy()
    np.testing.assert_allclose(c32, ref, rtol=1e-4, atol=1e-4 * max(np.abs(ref).max(), 1e-6))
    c = g.flatmm_a16w16(a, bs, n).float().cpu().numpy()
    assert (np.abs(c - ref) <= 1e-2 * np.abs(ref) + 1e-2).all()


def test_flat_gemm_exact_integers_and_decode_shape(orc):
    m, n, k = 16, 16384, 7168
    gen = torch.Generator(device="cuda"); gen.manual_seed(8)
    a = torch.randint(-4, 5, (m, k), generator=gen, device="cuda").to(torch.bfloat16)
    b = torch.randint(-4, 5, (n, k), generator=gen, device="cuda").to(torch.bfloat16)
    want = a.float() @ b.float().T
    assert torch.equal(g.flatmm_a16w16(a, g.preshuffle_b_bf16_device(b), n, c_dtype=g.FP32), want)


@pytest.mark.parametrize("m", [17, 33, 48, 49, 64, 80, 128])
@pytest.mark.parametrize("n,batch", [(144, 2), (288, 57)])      # two / four weight tiles per workgroup
def test_flat_gemm_row_groups_exact(m, n, batch):
    """M > 16: up to four groups of 16 rows share one pass over the weights (rows staged through LDS)."""
    k = 160                                                      # 320 bytes a row: an odd number of 64-byte K blocks
    gen = torch.Generator(device="cuda"); gen.manual_seed(900 + m + n)
    a = torch.randint(-4, 5, (batch, m, k), generator=gen, device="cuda").to(torch.bfloat16)
    b = torch.randint(-4, 5, (batch, n, k), generator=gen, device="cuda").to(torch.bfloat16)
    bs = torch.stack([g.preshuffle_b_bf16_device(b[i]) for i in range(batch)])
    got = g.flatmm_a16w16(a, bs, n, c_dtype=g.FP32)
    assert torch.equal(got, torch.einsum("bmk,bnk->bmn", a.float(), b.float()))


@pytest.mark.parametrize("m", [1, 16, 40, 64, 100, 128])
@pytest.mark.parametrize("n,batch", [(144, 2), (288, 57)])
def test_skinny_gemm_on_row_major_weights_exact(m, n, batch):
    """a16w16_gemm with at most 128 rows on row-major weights runs the flat kernel (weight rows staged through LDS)."""
    k = 160
    gen = torch.Generator(device="cuda"); gen.manual_seed(950 + m + n)
    a = torch.randint(-4, 5, (batch, m, k), generator=gen, device="cuda").to(torch.bfloat16)
    b = torch.randint(-4, 5, (batch, n, k), generator=gen, device="cuda").to(torch.bfloat16)
    got = g.gemm_a16w16(a, b, c_dtype=g.FP32)
    assert torch.equal(got, torch.einsum("bmk,bnk->bmn", a.float(), b.float()))
    # the same bits as the flat entry point on shuffled weights
    bs = torch.stack([g.preshuffle_b_bf16_device(b[i]) for i in range(batch)])
    assert torch.equal(got, g.flatmm_a16w16(a, bs, n, c_dtype=g.FP32))
