"""GPU parity of the skinny-M flatmm over pre-shuffled weights."""
import numpy as np
import pytest

import datagen
import gcnasm_amd as g
from gpu_util import assert_close, assert_fp32_accurate, exact64, run_flatmm

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [(16, 256, 512), (16, 1024, 7168), (5, 48, 192), (33, 128, 256), (16, 16, 64)])
def test_flatmm_rowcol(orc, shape):
    m, n, k = shape
    a, b, sa, sb = datagen.row_col(m, n, k, seed=800 + n)
    bs = g.preshuffle_b(b)
    want = orc.flatmm_ref(a, bs, sa, sb, n)
    assert (want == orc.gemm_ref(a, b, sa, sb, orc.ROWCOL)).all()
    assert_close(run_flatmm(a, bs, sa, sb, n), want, f"flatmm {shape}")
    assert_fp32_accurate(run_flatmm(a, bs, sa, sb, n, c_dtype=g.FP32), *exact64(orc, a, b, sa, sb, g.ROWCOL))


def test_flatmm_exact_integers(orc):
    m, n, k = 16, 512, 1024
    a, b = datagen.small_ints(m, n, k, seed=31)
    want = orc.decode(a).astype(np.int64) @ orc.decode(b).astype(np.int64).T
    got = run_flatmm(a, g.preshuffle_b(b), np.ones(m, np.float32), np.ones(n, np.float32), n, c_dtype=g.FP32)
    assert (got == want).all()
    got = run_flatmm(a, g.preshuffle_b(b), np.ones(1, np.float32), np.ones(1, np.float32), n, mode=g.TENSOR,
                     c_dtype=g.FP32)
    assert (got == want).all()
