"""torch.ops.mi355_a8w8.*: shape-only implementations on the CPU (meta tensors), the real ones on the GPU."""
import numpy as np
import pytest
import torch

import gcnasm_amd as g


def test_fake_implementations_propagate_shapes():
    g.register_torch_ops()
    g.register_torch_ops()                                  # idempotent
    a = torch.empty((300, 512), dtype=torch.uint8, device="meta")
    b = torch.empty((200, 512), dtype=torch.uint8, device="meta")
    s = torch.empty((1,), dtype=torch.float32, device="meta")
    c = torch.ops.mi355_a8w8.gemm(a, b, s, s, g.TENSOR, False)
    assert c.shape == (300, 200) and c.dtype == torch.bfloat16
    c = torch.ops.mi355_a8w8.gemm(a.expand(2, 300, 512), b.expand(2, 200, 512), s, s, g.TENSOR, True)
    assert c.shape == (2, 300, 200) and c.dtype == torch.float32
    c = torch.ops.mi355_a8w8.flatmm(a[:16], b.reshape(-1), s, s, 200, g.ROWCOL, False)
    assert c.shape == (16, 200)
    x = torch.empty((256, 1024), dtype=torch.float32, device="meta")
    for mode, gr, shape, dt in ((g.TENSOR, 1, (1,), torch.float32), (g.ROWCOL, 1, (256,), torch.float32),
                                (g.BLOCK, 1, (8, 256), torch.float32), (g.BLOCK, 128, (2, 8), torch.float32),
                                (g.MX, 1, (256, 32), torch.uint8), (g.MX_TILED, 1, (g.mx_tiled_bytes(256, 1024),), torch.uint8)):
        q, sc = torch.ops.mi355_a8w8.quantize(x, mode, gr)
        assert q.shape == (256, 1024) and q.dtype == torch.uint8 and sc.shape == shape and sc.dtype == dt
    h = torch.empty((64, 128), dtype=torch.bfloat16, device="meta")
    assert torch.ops.mi355_a8w8.gemm_a16w16(h, h, True).shape == (64, 64)
    q, sc = torch.ops.mi355_a8w8.quantize_mxfp4(x, True)
    assert q.shape == (256, 512) and sc.shape == (g.mx_tiled_bytes(256, 1024),)
    q2, sc2 = torch.ops.mi355_a8w8.quantize_mxfp4(x, False)
    assert sc2.shape == (256, 32)
    assert torch.ops.mi355_a8w8.gemm_a4w4(q, q[:64], sc, sc, g.MX_TILED, False).shape == (256, 64)
    c = torch.ops.mi355_a8w8.flatmm_a4w4(q[:16], q.reshape(-1), sc, sc, 256, True)
    assert c.shape == (16, 256) and c.dtype == torch.float32


@pytest.mark.gpu
def test_operators_run_the_library(orc):
    g.register_torch_ops()
    gen = torch.Generator(device="cuda"); gen.manual_seed(3)
    xa = torch.randn((256, 512), generator=gen, device="cuda")
    xb = torch.randn((384, 512), generator=gen, device="cuda")
    qa, sa = torch.ops.mi355_a8w8.quantize(xa, g.ROWCOL, 1)
    qb, sb = torch.ops.mi355_a8w8.quantize(xb, g.ROWCOL, 1)
    c = torch.ops.mi355_a8w8.gemm(qa, qb, sa, sb, g.ROWCOL, True)
    ref = orc.gemm_ref(qa.cpu().numpy(), qb.cpu().numpy(), sa.cpu().numpy(), sb.cpu().numpy(), orc.ROWCOL)
    np.testing.assert_allclose(c.cpu().numpy(), ref, rtol=1e-3, atol=1e-3 * np.abs(ref).max())
    assert torch.equal(c, g.gemm(qa, qb, sa, sb, g.ROWCOL, c_dtype=g.FP32))
    cf = torch.ops.mi355_a8w8.flatmm(qa[:16].contiguous(), g.preshuffle_b_device(qb), sa[:16].contiguous(), sb, 384, g.ROWCOL, True)
    np.testing.assert_allclose(cf.cpu().numpy(), ref[:16], rtol=1e-3, atol=1e-3 * np.abs(ref).max())
    h = xa.to(torch.bfloat16)
    assert torch.equal(torch.ops.mi355_a8w8.gemm_a16w16(h, h, False), g.gemm_a16w16(h, h))
    q4a, s4a = torch.ops.mi355_a8w8.quantize_mxfp4(xa[:16].contiguous(), True)
    q4b, s4b = torch.ops.mi355_a8w8.quantize_mxfp4(xb, True)
    c4 = torch.ops.mi355_a8w8.gemm_a4w4(q4a, q4b, s4a, s4b, g.MX_TILED, True)
    f4 = torch.ops.mi355_a8w8.flatmm_a4w4(q4a, g.preshuffle_b_device(q4b), s4a, s4b, 384, True)
    assert torch.equal(c4, g.gemm_a4w4(q4a, q4b, s4a, s4b, c_dtype=g.FP32))
    np.testing.assert_allclose(f4.cpu().numpy(), c4.cpu().numpy(), rtol=1e-4, atol=1e-3)
