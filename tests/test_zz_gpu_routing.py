"""Kernel choice for skinny problems (M <= 128) on shuffled weights: the entry points pick between the flat GEMM
and the MFMA tile kernels with a cost model (prefer_flat in the library).  For cells of the table that model was
fitted to, both sides are timed through a8w8_route_override and the model's own choice has to be within 10% of
the faster one.  The two sides must also agree on the result."""
import pytest
import torch

import gcnasm_amd as g

pytestmark = pytest.mark.gpu

FLAT, DENSE, MODEL = 1, 2, 0


def _time_us(fn, launches=30, regions=5):
    for i in range(12):
        fn(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(regions):
        e0.record()
        for i in range(launches):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) / launches)
    return best * 1e3


@pytest.mark.parametrize("mode", [g.ROWCOL, g.MX_TILED], ids=["rowcol", "mxfp8"])
@pytest.mark.parametrize("n,k", [(16384, 7168), (8192, 8192), (28672, 4096)])
def test_model_takes_a_side_within_ten_percent_of_the_faster(n, k, mode):
    L = g.lib()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(n + k)
    xb = torch.randn((n, k), generator=gen, device="cuda")
    copies = -(-(320 << 20) // (n * k))                      # rotate more weights than the 256 MB cache holds: they come from memory
    if mode == g.ROWCOL:
        qb, sb = g.quantize(xb, g.ROWCOL)
    else:
        qb, eb = g.quantize(xb, g.MX)
        sb = g.mx_tile_scales(eb)
    weights = [g.preshuffle_b_device(qb.clone()) for _ in range(copies)]
    del xb
    report = []
    try:
        for m in (16, 64, 96, 128):
            xa = torch.randn((m, k), generator=gen, device="cuda")
            if mode == g.ROWCOL:
                qa, sa = g.quantize(xa, g.ROWCOL)
            else:
                qa, ea = g.quantize(xa, g.MX)
                sa = g.mx_tile_scales(ea)
            c = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")

            def launch(i):
                g.gemm(qa, weights[i % copies], sa, sb, mode, c=c, n=n)

            took, out = {}, {}
            for attempt in range(3):      # a cell that misses is timed again (all three sides): clocks drift between regions
                for side in (FLAT, DENSE, MODEL):
                    assert L.a8w8_route_override(side) >= 0
                    took[side] = _time_us(launch)
                    launch(0)
                    torch.cuda.synchronize()
                    out[side] = c.float().clone()
                if took[MODEL] <= 1.10 * min(took[FLAT], took[DENSE]):
                    break
            L.a8w8_route_override(MODEL)
            # the same product from both kernel families (bf16 outputs of two fp32 summation orders)
            assert torch.allclose(out[FLAT], out[DENSE], rtol=2e-2, atol=2e-2), f"m={m}"
            report.append((m, took[FLAT], took[DENSE], took[MODEL]))
            print(f"{n}x{k} m={m} mode={mode}: flat {took[FLAT]:.1f} us, dense {took[DENSE]:.1f} us, model {took[MODEL]:.1f} us", flush=True)
    finally:
        L.a8w8_route_override(MODEL)
    for m, flat, dense, model in report:
        assert model <= 1.10 * min(flat, dense), f"{n}x{k} m={m}: model {model:.1f} us, flat {flat:.1f} us, dense {dense:.1f} us"


def test_override_is_validated_and_reported():
    L = g.lib()
    assert L.a8w8_route_override(7) == -6
    args = g.raw_gemm_args(1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, 16, 16384, 7168, g.ROWCOL, b_preshuffled=1)
    try:
        assert L.a8w8_route_override(DENSE) == MODEL
        assert g.kernel_name(args) == "gemm_a8w8_tile128"
        assert L.a8w8_route_override(FLAT) == DENSE
        assert g.kernel_name(args) == "flatmm_a8w8"
    finally:
        L.a8w8_route_override(MODEL)
    assert g.kernel_name(args) == "flatmm_a8w8"
