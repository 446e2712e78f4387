"""GPU parity at the benchmark configurations' full sizes.  The oracle checks a slab of rows plus
random probes (the whole output would take minutes on the CPU); whole-output checks use
properties that need no oracle: exact scaling by powers of two and row-permutation equivariance."""
import numpy as np
import pytest
import torch

import datagen
import gcnasm_amd as g
from gpu_util import MFMA_ACC_ERR, assert_close, dev, exact64

pytestmark = pytest.mark.gpu


def _check_slab_and_probes(orc, c, a, b, sfa, sfb, mode, rows=16, nprobe=4096, seed=1):
    """|C - Cref| <= 1e-2*|Cref| + 1e-2 on the first `rows` rows and on random (i, j) probes; the few
    cancellation-dominated outputs the MFMA's accumulation error can push past the bound (MX inputs
    only) must stay within MFMA_ACC_ERR of sum|a||b|s and be under 0.1%."""
    m, n = c.shape
    ref = orc.gemm_ref(a, b, sfa, sfb, mode, rows=(0, rows))
    got = c[:rows]
    rng = np.random.Generator(np.random.Philox(seed))
    pi = rng.integers(0, m, nprobe).astype(np.int32)
    pj = rng.integers(0, n, nprobe).astype(np.int32)
    pref = orc.gemm_probe(a, b, sfa, sfb, mode, pi, pj)
    got_all = np.concatenate([got.ravel(), c[pi, pj]])
    ref_all = np.concatenate([ref.ravel(), pref])
    miss = ~(np.abs(got_all - ref_all) <= 1e-2 * np.abs(ref_all) + 1e-2)
    if mode == orc.MX and miss.any():
        assert miss.mean() <= 1e-3, f"{miss.sum()} of {miss.size} outside tolerance"
        # magnitude yardstick for the slab rows only (probes that miss are re-checked through their row)
        idx = np.nonzero(miss)[0]
        for t in idx:
            if t < ref.size:
                i, j = divmod(int(t), n)
            else:
                i, j = int(pi[t - ref.size]), int(pj[t - ref.size])
            av = orc.decode(a[i]).astype(np.float64).reshape(-1, 32)
            bv = orc.decode(b[j]).astype(np.float64).reshape(-1, 32)
            s = np.exp2(sfa[i].astype(np.float64) - 127) * np.exp2(sfb[j].astype(np.float64) - 127)
            exact = ((av * bv).sum(axis=1) * s).sum()
            mag = ((np.abs(av) * np.abs(bv)).sum(axis=1) * s).sum()
            assert abs(got_all[t] - exact) <= MFMA_ACC_ERR * mag + 2.0 ** -8 * abs(exact), (i, j, got_all[t], exact)
    else:
        assert not miss.any(), f"{miss.sum()} of {miss.size} outside tolerance"


def test_config2_rowcol_4096(orc):
    a, b, sa, sb = datagen.row_col(4096, 4096, 4096)
    c = g.gemm(dev(a), dev(b), dev(sa), dev(sb), g.ROWCOL).float().cpu().numpy()
    _check_slab_and_probes(orc, c, a, b, sa, sb, orc.ROWCOL)


def test_config3_block_scale_4096x7168x2048(orc):
    a, b, sfa, sfb = datagen.block_scaled(4096, 7168, 2048)
    c = g.gemm(dev(a), dev(b), dev(sfa), dev(sfb), g.BLOCK).float().cpu().numpy()
    _check_slab_and_probes(orc, c, a, b, sfa, sfb, orc.BLOCK)


def test_config4_mxfp8_8192_and_whole_output_properties(orc):
    m = n = k = 8192
    a, b, ea, eb = datagen.mx(m, n, k)
    da, db, dea, deb = dev(a), dev(b), dev(ea), dev(eb)
    c = g.gemm(da, db, dea, deb, g.MX)
    _check_slab_and_probes(orc, c.float().cpu().numpy(), a, b, ea, eb, orc.MX, rows=8, nprobe=2048)
    # doubling every A-side scale doubles every output exactly (a power of two survives bf16 rounding)
    c2 = g.gemm(da, db, dea + 1, deb, g.MX)
    assert torch.equal(c2.float(), 2 * c.float())
    # permuting the rows of A (with their scales) permutes the rows of C bit for bit
    perm = torch.randperm(m, generator=torch.Generator().manual_seed(3)).cuda()
    cp = g.gemm(da[perm].contiguous(), db, dea[perm].contiguous(), deb, g.MX)
    assert torch.equal(cp, c[perm])


def test_config5_flatmm_16x16384x7168(orc):
    m, n, k = 16, 16384, 7168
    a, b, sa, sb = datagen.row_col(m, n, k, seed=datagen.SEED_BASE + 5)
    bs = g.preshuffle_b(b)
    assert (bs == orc.preshuffle_b(b)).all()
    c = g.flatmm(dev(a), dev(bs), dev(sa), dev(sb), n).float().cpu().numpy()
    ref = orc.gemm_ref(a, b, sa, sb, orc.ROWCOL)
    assert (np.abs(c - ref) <= 1e-2 * np.abs(ref) + 1e-2).all()
    # the device-side shuffle feeds the same kernel to the same result
    c2 = g.flatmm(dev(a), g.preshuffle_b_device(dev(b)), dev(sa), dev(sb), n).float().cpu().numpy()
    assert (c2 == c).all()


def test_more_tiles_than_compute_units(orc):
    """17 x 17 = 289 tiles: some workgroups of the persistent kernel run two tiles back to back."""
    m = n = 4352
    k = 384
    a, b, sa, sb = datagen.row_col(m, n, k, seed=901)
    c = g.gemm(dev(a), dev(b), dev(sa), dev(sb), g.ROWCOL).float().cpu().numpy()
    _check_slab_and_probes(orc, c, a, b, sa, sb, orc.ROWCOL, rows=8, nprobe=8192)
    a, b, ea, eb = datagen.mx(m, n, k, seed=902)
    c = g.gemm(dev(a), dev(b), dev(ea), dev(eb), g.MX).float().cpu().numpy()
    _check_slab_and_probes(orc, c, a, b, ea, eb, orc.MX, rows=8, nprobe=8192)
    # exact integers over the same shape: every tile, every K step, bit for bit
    a, b = datagen.small_ints(m, n, k, seed=903, lo=-2, hi=2)
    want = torch.from_numpy(orc.decode(a)).cuda() @ torch.from_numpy(orc.decode(b)).cuda().T
    got = g.gemm(dev(a), dev(b), dev(np.ones(m, np.float32)), dev(np.ones(n, np.float32)), g.ROWCOL, c_dtype=g.FP32)
    assert torch.equal(got, want)


@pytest.mark.parametrize("mode", [g.ROWCOL, g.MX])
def test_batched_persistent(orc, mode):
    batch, m, n, k = 3, 300, 520, 384
    gen = datagen.row_col if mode == g.ROWCOL else datagen.mx
    per = [gen(m, n, k, seed=950 + i) for i in range(batch)]
    a, b, sa, sb = (np.stack([p[i] for p in per]) for i in range(4))
    c = g.gemm(dev(a), dev(b), dev(sa), dev(sb), mode, c_dtype=g.FP32).cpu().numpy()
    for i in range(batch):
        ref = orc.gemm_ref(a[i], b[i], sa[i], sb[i], mode)
        if mode == g.MX:
            # wide-range inputs: outputs that cancel to almost zero are judged against float64 (gpu_util.assert_close)
            exact, mag = exact64(orc, a[i], b[i], sa[i], sb[i], mode)
            assert_close(c[i], ref, f"batch entry {i}", exact=exact, mag=mag)
        else:
            assert datagen.tolerance_ok(c[i], ref).all(), i
        np.testing.assert_allclose(c[i], ref, rtol=2e-3, atol=2e-3 * np.abs(ref).max())
