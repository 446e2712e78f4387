"""The entry points under HIP graph capture: the library allocates nothing and enqueues kernels only, so a
serving loop can record quantise -> scale re-order -> GEMM once and replay it.  Every replay is checked against
the eager result on fresh inputs, with the program's own eager work between the replays."""
import numpy as np
import pytest
import torch

import gcnasm_amd as g

pytestmark = pytest.mark.gpu


def _fresh(shape, seed):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    return torch.randn(shape, generator=gen, device="cuda")


@pytest.mark.parametrize("m,n,k", [(512, 768, 1024), (4096, 4608, 512)])      # 128-tile kernel / four-wave kernel
def test_quantise_reorder_gemm_replays(m, n, k):
    xa, xb = _fresh((m, k), 1), _fresh((n, k), 2)
    qa = torch.empty((m, k), dtype=torch.uint8, device="cuda")
    qb = torch.empty((n, k), dtype=torch.uint8, device="cuda")
    ea = torch.empty((m, k // 32), dtype=torch.uint8, device="cuda")
    eb = torch.empty((n, k // 32), dtype=torch.uint8, device="cuda")
    ta = torch.empty(g.mx_tiled_bytes(m, k), dtype=torch.uint8, device="cuda")
    tb = torch.empty(g.mx_tiled_bytes(n, k), dtype=torch.uint8, device="cuda")
    c = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    L = g.lib()

    def pipeline():
        s = g.api._stream()
        assert L.a8w8_quantize(xa.data_ptr(), m, k, k, qa.data_ptr(), ea.data_ptr(), g.MX, 1, s) == 0
        assert L.a8w8_quantize(xb.data_ptr(), n, k, k, qb.data_ptr(), eb.data_ptr(), g.MX, 1, s) == 0
        assert L.a8w8_mx_tile_scales_ab(ea.data_ptr(), m, k // 32, ta.data_ptr(), eb.data_ptr(), n, k // 32, tb.data_ptr(), k, s) == 0
        g.gemm(qa, qb, ta, tb, g.MX_TILED, c=c)

    pipeline()                                  # eager once: first-use set-up happens outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            pipeline()
    torch.cuda.synchronize()
    for rep in range(3):
        xa.copy_(_fresh((m, k), 10 + rep))
        xb.copy_(_fresh((n, k), 20 + rep))
        graph.replay()
        torch.cuda.synchronize()
        got = c.clone()
        c.zero_()
        pipeline()
        torch.cuda.synchronize()
        assert torch.equal(got, c), f"replay {rep} differs from the eager result"
        ref = xa @ xb.T
        assert (got.float() - ref).abs().max() <= 0.08 * ref.abs().max()      # FP8 quantisation error, not a parity bound


def test_per_tensor_quantiser_replays():
    """The per-tensor quantiser is four launches around one device-side maximum: replays must start from a clean one."""
    rows, k = 300, 1024
    x = _fresh((rows, k), 3)
    q = torch.empty((rows, k), dtype=torch.uint8, device="cuda")
    s = torch.empty(1, dtype=torch.float32, device="cuda")
    L = g.lib()

    def run():
        assert L.a8w8_quantize(x.data_ptr(), rows, k, k, q.data_ptr(), s.data_ptr(), g.TENSOR, 1, g.api._stream()) == 0

    run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            run()
    torch.cuda.synchronize()
    for rep in range(3):
        x.copy_(_fresh((rows, k), 30 + rep) * (0.25 if rep == 1 else 4.0))      # a smaller maximum after a larger one
        graph.replay()
        torch.cuda.synchronize()
        got_q, got_s = q.clone(), s.clone()
        run()
        torch.cuda.synchronize()
        assert torch.equal(got_q, q) and torch.equal(got_s, s)
        assert np.isclose(float(got_s[0]), float(x.abs().max()) / 448.0, rtol=1e-6)


@pytest.mark.parametrize("m", [16, 48, 128])      # fragments gathered from memory / rows staged through LDS / two row-group sets
def test_flat_gemm_replays(m):
    """Decode step under capture: quantise the activations, flat GEMM over shuffled weights."""
    n, k = 2048, 1024
    xa, xb = _fresh((m, k), 5), _fresh((n, k), 6)
    qb, sb = g.quantize(xb, g.ROWCOL)
    bs = g.preshuffle_b_device(qb)
    qa = torch.empty((m, k), dtype=torch.uint8, device="cuda")
    sa = torch.empty(m, dtype=torch.float32, device="cuda")
    c = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    L = g.lib()

    def step():
        assert L.a8w8_quantize(xa.data_ptr(), m, k, k, qa.data_ptr(), sa.data_ptr(), g.ROWCOL, 1, g.api._stream()) == 0
        g.flatmm(qa, bs, sa, sb, n, c=c)

    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.synchronize()
    for rep in range(3):
        xa.copy_(_fresh((m, k), 40 + rep))
        graph.replay()
        torch.cuda.synchronize()
        got = c.clone()
        c.zero_()
        step()
        torch.cuda.synchronize()
        assert torch.equal(got, c), f"replay {rep} differs from the eager result"
        ref = xa @ xb.T
        assert (got.float() - ref).abs().max() <= 0.08 * ref.abs().max()      # FP8 quantisation error, not a parity bound
