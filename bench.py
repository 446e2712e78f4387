#!/usr/bin/env python3
"""Benchmark of the A8W8 FP8 GEMM path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--no-extra]

One "step" is one pass of the hot path over one batch of synthetic, already-quantised
inputs resident in HBM.  The headline workload is the MXFP8 GEMM M=N=K=8192 (E4M3 elements,
one E8M0 exponent per 32 K-elements in row-major [rows][K/32] arrays, bf16 out).  Its step is
two launches: both scale arrays are re-ordered into the tiled layout (a8w8_mx_tile_scales_ab)
and the GEMM runs on the tiled scales; the GEMM launch alone (scales already tiled, as a
quantiser can emit them) and the one-launch path on row-major scales are timed beside it.
The other configurations and the M=16 flatmm are timed afterwards and reported in the same
JSON line under "other_workloads".
Timing uses HIP events recorded on the stream the kernels are launched on, W untimed
warm-up launches, then exactly K timed launches.  The chip's clocks take a few hundred
milliseconds of load to settle, so every timed workload is preceded by a time-based run of
the same launches that is counted neither in W nor in K; for the headline workload the same
W + K protocol is also run once before that, on the cold chip, and reported beside the
steady number ("first_region").  The CPU baseline is the oracle (a port of the reference's
host GEMM) timed on a bounded slab of each configuration.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "FP8 GEMM TFLOPS & % gfx950 FP8 MFMA peak; HBM GB/s for M=16 flatmm"
PEAK_FP8_TFLOPS = 5000.0      # MI355X dense FP8 MFMA, published
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E, published
PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA, published
PEAK_FP4_TFLOPS = 10100.0     # MI355X dense FP4 MFMA, published


def measured_traffic():
    """Bytes that crossed the L2 <-> fabric boundary per launch of each workload's dominant kernel, as the tracked
    summary of the two rocprofv3 --pmc runs of this file states them (FETCH_SIZE and WRITE_SIZE, each scaled by what
    the counter reads for a device copy of known size); None for a workload the summary does not list."""
    import re
    path = os.path.join(ROOT, "profiles", "traffic_fetch_write.md")
    out = {}
    try:
        for line in open(path):
            m = re.match(r"\s*traffic_bytes_per_launch\s+(\S+)\s*=\s*([0-9.eE+]+)", line)
            if m:
                out[m.group(1)] = float(m.group(2))
    except OSError:
        pass
    return out


WORKLOADS = {
    # name: (mode, m, n, k, algorithmic bytes per launch)
    "mxfp8_8192": ("mx", 8192, 8192, 8192, 272629760),
    "rowcol_4096": ("rowcol", 4096, 4096, 4096, 67141632),
    "block_4096x7168x2048": ("block", 4096, 7168, 2048, 82054656),
    "tensor_256": ("tensor", 256, 256, 256, 262152),
    "flatmm_16x16384x7168": ("flat", 16, 16384, 7168, 118145088),
    # the bf16 sibling (a16w16_gemm), priced against the dense bf16 peak
    "a16w16_4096": ("bf16", 4096, 4096, 4096, 100663296),
    # MXFP4 (a4w4_gemm, tiled scales), priced against the dense FP4 peak
    "mxfp4_8192": ("f4", 8192, 8192, 8192, 205520896),
    # short and wide (a prefill chunk of 256 tokens over a 64 MiB weight): between the flat GEMM's M <= 128 and the
    # 256-row tiles; A 2 MiB + B 64 MiB + C 4 MiB + scales
    "gemm_rowcol_256x8192x8192": ("rowcol", 256, 8192, 8192, 73434112),
    # the two pipelined kernels on one scale mode: 64 K steps run on the four-wave kernel, 65 (an odd count) on the
    # eight-wave kernel with two waves per SIMD; compared per K step
    "tensor_8192": ("tensor", 8192, 8192, 8192, 268435464),
    "tensor_8192x8192x8320": ("tensor", 8192, 8192, 8320, 270532616),
    # the 128-tile kernel's variants: one tile per compute unit (four LDS stages), two per compute unit (two stages)
    "rowcol_2048": ("rowcol", 2048, 2048, 2048, 16793600),
    "rowcol_2048x4096x2048": ("rowcol", 2048, 4096, 2048, 29384704),
}
# selectable with --workload, not part of the default run's secondary workloads
SELECT_ONLY = {"tensor_8192", "tensor_8192x8192x8320", "rowcol_2048", "rowcol_2048x4096x2048"}
# workloads whose weights would stay in the 256 MB Infinity Cache between launches: timed over rotating copies of B
ROTATE_B = {"gemm_rowcol_256x8192x8192": 5}


def make_inputs(name, torch, g, seed):
    """Synthetic operands of the workload's shape, quantised on the GPU by the library's own
    front end (values N(0,1); the MX case multiplies each 32-block by 2^U(-4,4))."""
    mode, m, n, k, _ = WORKLOADS[name]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)

    def normal(rows):
        return torch.randn((rows, k), generator=gen, device="cuda", dtype=torch.float32)

    if mode == "f4":
        a, sfa = g.quantize_mxfp4(normal(m), tiled=True)
        b, sfb = g.quantize_mxfp4(normal(n), tiled=True)
        return dict(a=a, b=b, sfa=sfa, sfb=sfb, mode=g.MX_TILED)
    if mode == "bf16":
        a = torch.randn((m, k), generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
        b = torch.randn((n, k), generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
        return dict(a=a, b=b, sfa=a, sfb=b, mode=g.TENSOR)
    if mode == "mx":
        out = []
        for rows in (m, n):
            x = normal(rows).view(rows, k // 32, 32)
            x = x * torch.exp2(torch.rand((rows, k // 32, 1), generator=gen, device="cuda") * 8 - 4)
            out.append(g.quantize(x.view(rows, k).contiguous(), g.MX))
            del x
        (a, sfa), (b, sfb) = out
        return dict(a=a, b=b, sfa=sfa, sfb=sfb, mode=g.MX)
    if mode == "block":
        a, sfa = g.quantize(normal(m), g.BLOCK, 1)
        b, sfb = g.quantize(normal(n), g.BLOCK, 128)
        return dict(a=a, b=b, sfa=sfa, sfb=sfb, mode=g.BLOCK)
    if mode == "tensor":
        a, sfa = g.quantize(normal(m), g.TENSOR)
        b, sfb = g.quantize(normal(n), g.TENSOR)
        return dict(a=a, b=b, sfa=sfa, sfb=sfb, mode=g.TENSOR)
    a, sfa = g.quantize(normal(m), g.ROWCOL)
    b, sfb = g.quantize(normal(n), g.ROWCOL)
    if mode == "flat":
        return dict(a=a, b=b, sfa=sfa, sfb=sfb, mode=g.ROWCOL, bshuf=g.preshuffle_b_device(b))
    return dict(a=a, b=b, sfa=sfa, sfb=sfb, mode=g.ROWCOL)


def time_launches(torch, fn, steps, warmup):
    """Average launch duration in ms: W warm-up launches, then K launches between two HIP
    events on the current stream (the stream the library is handed)."""
    for _ in range(warmup):
        fn(0)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return e0.elapsed_time(e1) / steps, wall_ms / steps


CONDITION_S = 0.5      # load applied before a timed region, counted in neither W nor K


def condition_clocks(torch, fn, seconds=CONDITION_S):
    """Runs the workload's own launches for `seconds` of wall time so that the timed region that follows sees
    the clocks the chip sustains under this load rather than the ramp from idle."""
    t0 = time.perf_counter()
    i = 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn(i)
            i += 1
        torch.cuda.synchronize()


def time_steady(torch, fn, steps, warmup):
    """The headline protocol: conditioning, then W warm-up launches and exactly K timed ones."""
    condition_clocks(torch, fn)
    return time_launches(torch, fn, steps, warmup)


def time_best_of(torch, fn, steps, warmup, rounds=3):
    """For the secondary workloads: bring the clocks up with at least 100 ms of warm-up launches,
    then report the best of `rounds` timed regions of `steps` launches each."""
    condition_clocks(torch, fn, 0.1)
    best = None
    for _ in range(rounds):
        r = time_launches(torch, fn, steps, warmup)
        if best is None or r[0] < best[0]:
            best = r
    return best


def run_workload(name, torch, g, steps, warmup, seed, headline=True, operands="as_configured"):
    mode, m, n, k, abytes = WORKLOADS[name]
    inp = make_inputs(name, torch, g, seed)
    if operands == "zeros":
        # the same launch on operands that toggle nothing: what the schedule alone allows (a measurement aid)
        inp["a"].zero_()
        inp["b"].zero_()
    elif operands == "random_bytes":
        # full-entropy operand bytes (the two NaN codes of E4M3 mapped to finite values)
        for t in (inp["a"], inp["b"]):
            r = torch.randint(0, 256, t.shape, device="cuda", dtype=torch.int16).to(torch.uint8)
            r[(r & 0x7F) == 0x7F] = 0x3C
            t.copy_(r)
            del r
    flops = 2.0 * m * n * k
    c = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    res = {"workload": name, "m": m, "n": n, "k": k}
    res["kernel"] = "flatmm_a8w8" if mode == "flat" else None
    import ctypes
    L = g.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def args_for(b_tensor, preshuffled):
        # the C argument block is filled once; the timed loop is only the C-ABI call
        return g.raw_gemm_args(inp["a"].data_ptr(), b_tensor.data_ptr(), c.data_ptr(), inp["sfa"].data_ptr(),
                               inp["sfb"].data_ptr(), m, n, k, inp["mode"], g.BF16, b_preshuffled=preshuffled)

    if mode == "flat":
        # B (117 MB) fits the 256 MB Infinity Cache: rotate four copies so every launch reads HBM
        copies = [inp["bshuf"]] + [inp["bshuf"].clone() for _ in range(3)]
        flat_args = [ctypes.byref(args_for(x, 1)) for x in copies]
        keep = [a._obj for a in flat_args]   # noqa: F841  (keeps the structs alive)

        def fn_rot(i):
            if L.a8w8_flatmm(flat_args[i & 3], stream) != 0:
                raise RuntimeError("a8w8_flatmm failed")

        def fn_same(i):
            if L.a8w8_flatmm(flat_args[0], stream) != 0:
                raise RuntimeError("a8w8_flatmm failed")

        timer = time_steady if headline else time_best_of
        ms, wall = timer(torch, fn_rot, steps, warmup)
        ms_same, _ = timer(torch, fn_same, steps, warmup)
        res.update(ms_per_launch=ms, wall_ms_per_launch=wall, gbs=abytes / ms / 1e6, gbs_same_buffer=abytes / ms_same / 1e6,
                   tflops=flops / ms / 1e9, frac_hbm_peak=abytes / ms / 1e6 / PEAK_HBM_GBS,
                   note="four rotating copies of B (470 MB) defeat the 256 MB Infinity Cache; gbs_same_buffer re-reads one copy")
        # the same launches replayed from one HIP graph: what is left of the gap between back-to-back launches
        graph_steps = 64
        side = torch.cuda.Stream()
        side_stream = ctypes.c_void_p(side.cuda_stream)
        with torch.cuda.stream(side):
            for i in range(4):
                L.a8w8_flatmm(flat_args[i], side_stream)
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                cap = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
                for i in range(graph_steps):
                    if L.a8w8_flatmm(flat_args[i & 3], cap) != 0:
                        raise RuntimeError("a8w8_flatmm failed under capture")
        ms_graph, _ = time_best_of(torch, lambda i: graph.replay(), max(2, steps // 16), 2)
        ms_graph /= graph_steps
        res.update(ms_per_launch_in_graph=ms_graph, gbs_in_graph=abytes / ms_graph / 1e6,
                   frac_hbm_peak_in_graph=abytes / ms_graph / 1e6 / PEAK_HBM_GBS,
                   graph_note=f"{graph_steps} launches (rotating B) captured in one HIP graph and replayed")
        # yardstick: what a kernel that only reads the same rotating buffers gets on this box
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        probe_args = [(ctypes.c_void_p(x.data_ptr()), x.numel()) for x in copies]

        def fn_probe(i):
            ptr, nbytes = probe_args[i & 3]
            if L.a8w8_hbm_read_probe(ptr, nbytes, ctypes.c_void_p(sink.data_ptr()), stream) != 0:
                raise RuntimeError("a8w8_hbm_read_probe failed")

        ms_probe, _ = time_best_of(torch, fn_probe, steps, warmup)
        wbytes = copies[0].numel()
        res.update(achievable_read_gbs=wbytes / ms_probe / 1e6, achievable_read_ms=ms_probe,
                   frac_of_achievable_read=(abytes / ms) / (wbytes / ms_probe),
                   achievable_note="a8w8_hbm_read_probe: 16-byte non-temporal loads over the same four weight buffers, nothing else "
                                   "(after the reference's bandwidth_memread)")
        fn = fn_rot
    else:
        gemm_args = args_for(inp["b"], 0)
        gemm_ref_ = ctypes.byref(gemm_args)

        entry = L.a16w16_gemm if mode == "bf16" else L.a4w4_gemm if mode == "f4" else L.a8w8_gemm

        if name in ROTATE_B:
            b_copies = [inp["b"]] + [inp["b"].clone() for _ in range(ROTATE_B[name] - 1)]
            rot_structs = [args_for(x, 0) for x in b_copies]
            rot_refs = [ctypes.byref(x) for x in rot_structs]
            res["note"] = f"{len(b_copies)} rotating copies of B ({len(b_copies) * n * k >> 20} MiB): every launch reads its weights from HBM"
            res["frac_hbm_peak"] = None      # filled in below

            def fn_direct(i):
                if entry(rot_refs[i % len(rot_refs)], stream) != 0:
                    raise RuntimeError("gemm call failed")
        else:
            def fn_direct(i):
                if entry(gemm_ref_, stream) != 0:
                    raise RuntimeError("gemm call failed")

        fn = fn_direct
        timer = time_steady if headline else time_best_of
        if mode == "mx":
            # row-major scales in, tiled scales for the kernel: two re-ordering launches + the GEMM
            ta = torch.empty(g.mx_tiled_bytes(m, k), dtype=torch.uint8, device="cuda")
            tb = torch.empty(g.mx_tiled_bytes(n, k), dtype=torch.uint8, device="cuda")
            tiled_args = g.raw_gemm_args(inp["a"].data_ptr(), inp["b"].data_ptr(), c.data_ptr(), ta.data_ptr(),
                                         tb.data_ptr(), m, n, k, g.MX_TILED, g.BF16)
            tiled_ref = ctypes.byref(tiled_args)
            sfa_p, sfb_p, ta_p, tb_p = (ctypes.c_void_p(t.data_ptr()) for t in (inp["sfa"], inp["sfb"], ta, tb))

            def fn_gemm_only(i):
                if L.a8w8_gemm(tiled_ref, stream) != 0:
                    raise RuntimeError("a8w8_gemm failed")

            def fn(i):
                if (L.a8w8_mx_tile_scales_ab(sfa_p, m, k // 32, ta_p, sfb_p, n, k // 32, tb_p, k, stream) != 0
                        or L.a8w8_gemm(tiled_ref, stream) != 0):
                    raise RuntimeError("a8w8_mx_tile_scales_ab / a8w8_gemm failed")

            res["kernel"] = g.kernel_name(tiled_args)
            if headline:
                # the same protocol on the chip as it is found (idle clocks), reported beside the steady number
                first_ms, _ = time_launches(torch, fn, steps, warmup)
                res.update(first_region_ms_per_step=first_ms, first_region_tflops=flops / first_ms / 1e9)
            ms, wall = timer(torch, fn, steps, warmup)
            ms_gemm, _ = timer(torch, fn_gemm_only, steps, warmup)
            ms_direct, _ = timer(torch, fn_direct, steps, warmup)
            res.update(ms_gemm_kernel=ms_gemm, tflops_gemm_kernel=flops / ms_gemm / 1e9,
                       ms_row_major_scales_one_launch=ms_direct, tflops_row_major_scales_one_launch=flops / ms_direct / 1e9,
                       step="a8w8_mx_tile_scales_ab(sfa, sfb) + a8w8_gemm(MX_TILED)")
        else:
            res["kernel"] = ("gemm_a8w8_wide<bf16>" if mode == "bf16" else "gemm_a8w8_wide<mxfp4>" if mode == "f4"
                             else g.kernel_name(gemm_args))
            ms, wall = timer(torch, fn, steps, warmup)
        res.update(ms_per_launch=ms, wall_ms_per_launch=wall, tflops=flops / ms / 1e9, gbs=abytes / ms / 1e6)
        if mode == "bf16":
            res["frac_bf16_peak"] = flops / ms / 1e9 / PEAK_BF16_TFLOPS
        elif mode == "f4":
            res["frac_fp4_peak"] = flops / ms / 1e9 / PEAK_FP4_TFLOPS
        else:
            res["frac_fp8_peak"] = flops / ms / 1e9 / PEAK_FP8_TFLOPS
        if name in ROTATE_B:
            res["frac_hbm_peak"] = abytes / ms / 1e6 / PEAK_HBM_GBS
    fn(0)
    torch.cuda.synchronize()
    return res, inp, c


def run_quantizers(torch, g, steps, warmup, seed):
    """The quantisation front end on the headline's activation shape (fp32 8192 x 8192 in, E4M3 + scales out):
    HBM-bound byte work, priced against the HBM peak with each byte counted once."""
    import ctypes
    rows, k = 8192, 8192
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    x = torch.randn((rows, k), generator=gen, device="cuda", dtype=torch.float32)
    q = torch.empty((rows, k), dtype=torch.uint8, device="cuda")
    L = g.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = []
    for name, mode, scale_bytes in (("quantize_mx_tiled_8192", g.MX_TILED, g.mx_tiled_bytes(rows, k)),
                                    ("quantize_rowcol_8192", g.ROWCOL, rows * 4)):
        sc = torch.empty(scale_bytes, dtype=torch.uint8, device="cuda")
        xp, qp, sp = (ctypes.c_void_p(t.data_ptr()) for t in (x, q, sc))

        def fn(i):
            if L.a8w8_quantize(xp, rows, k, k, qp, sp, mode, 1, stream) != 0:
                raise RuntimeError("a8w8_quantize failed")

        ms, wall = time_best_of(torch, fn, steps, warmup)
        abytes = rows * k * 5 + scale_bytes
        out.append({"workload": name, "rows": rows, "k": k, "kernel": "a8w8_quantize", "ms_per_launch": ms,
                    "wall_ms_per_launch": wall, "algorithmic_bytes": abytes, "gbs": abytes / ms / 1e6,
                    "frac_hbm_peak": abytes / ms / 1e6 / PEAK_HBM_GBS,
                    "timing": "best of 3 regions of K launches after 100 ms of warm-up"})
    return out


# What the reference publishes for its own block-scale program (fp32 C, A~U[0,1), B~U[-.5,.5), scales~U[.8,1.2);
# opus_gemm/block_scale_gemm/README.md:111-115) and as the expected output of its flat program
# (opus_fmm/README.md:43-49, 2*16*4096*4096 flops), on MI355X.
REFERENCE_PUBLISHED = {"block_fp32_1024": 118.96, "block_fp32_2048": 616.77, "block_fp32_4096": 2237.77, "block_fp32_8192": 2710.24,
                       "block_fp32_16384": 2686.87, "flatmm_16x4096x4096": 20.64}


def run_reference_program_sizes(torch, g, steps, warmup, seed):
    """The reference's own programs at the sizes it publishes numbers for, with its inputs and its metric
    (2*M*N*K / average launch time): the ratio to the published TFlops is reported beside each."""
    import ctypes
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)

    def uniform(shape, lo, hi):
        return torch.rand(shape, generator=gen, device="cuda", dtype=torch.float32) * (hi - lo) + lo

    out = []
    for size in (1024, 2048, 4096, 8192, 16384):
        m = n = k = size
        a = g.cvt_f32_to_e4m3(uniform((m, k), 0.0, 1.0))
        torch.cuda.empty_cache()
        b = g.cvt_f32_to_e4m3(uniform((n, k), -0.5, 0.5))
        torch.cuda.empty_cache()
        sfa, sfb = uniform((k // 128, m), 0.8, 1.2), uniform((n // 128, k // 128), 0.8, 1.2)
        c = torch.empty((m, n), dtype=torch.float32, device="cuda")
        big_steps = steps if size < 16384 else max(5, steps // 5)      # 3.5 ms a launch: fewer of them
        # the argument block is filled once, as the reference's C++ program does: a launch through the tensor wrapper costs
        # the host 10 us, which is as long as the 1024-cube kernel runs
        args = g.raw_gemm_args(a.data_ptr(), b.data_ptr(), c.data_ptr(), sfa.data_ptr(), sfb.data_ptr(), m, n, k, g.BLOCK, c_dtype=g.FP32)
        ref, lib, stream = ctypes.byref(args), g.lib(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        assert lib.a8w8_gemm_blockscale(ref, stream) == 0
        ms, wall = time_best_of(torch, lambda i: lib.a8w8_gemm_blockscale(ref, stream), big_steps, min(warmup, big_steps))
        name = f"block_fp32_{size}"
        tf = 2.0 * m * n * k / ms / 1e9
        out.append({"workload": name, "m": m, "n": n, "k": k, "kernel": g.kernel_name(g.raw_gemm_args(
            1 << 12, 1 << 12, 1 << 12, 1 << 12, 1 << 12, m, n, k, g.BLOCK, c_dtype=g.FP32)), "ms_per_launch": ms,
            "wall_ms_per_launch": wall, "tflops": tf, "reference_published_tflops": REFERENCE_PUBLISHED[name],
            "vs_reference_published": tf / REFERENCE_PUBLISHED[name]})
        del a, b, sfa, sfb, c
        torch.cuda.empty_cache()
    m, n, k = 16, 4096, 4096
    a, sfa = g.quantize(torch.randn((m, k), generator=gen, device="cuda"), g.ROWCOL)
    b, sfb = g.quantize(torch.randn((n, k), generator=gen, device="cuda"), g.ROWCOL)
    bs = g.preshuffle_b_device(b)
    c = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    args = g.raw_gemm_args(a.data_ptr(), bs.data_ptr(), c.data_ptr(), sfa.data_ptr(), sfb.data_ptr(), m, n, k, g.ROWCOL, c_dtype=g.BF16,
                           b_preshuffled=1)
    ref, lib, stream = ctypes.byref(args), g.lib(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.a8w8_flatmm(ref, stream) == 0
    ms, wall = time_best_of(torch, lambda i: lib.a8w8_flatmm(ref, stream), steps, warmup)
    tf = 2.0 * m * n * k / ms / 1e9
    out.append({"workload": "flatmm_16x4096x4096", "m": m, "n": n, "k": k, "kernel": "flatmm_a8w8", "ms_per_launch": ms,
                "wall_ms_per_launch": wall, "tflops": tf, "reference_published_tflops": REFERENCE_PUBLISHED["flatmm_16x4096x4096"],
                "vs_reference_published": tf / REFERENCE_PUBLISHED["flatmm_16x4096x4096"],
                "note": "a launch from Python through ctypes still costs the host several us, which bounds this entry; the C++ "
                        "program tests/harness/flatmm_a8w8.exe -m 16 -n 4096 -k 4096 measures the kernel's own rate"})
    return out


def run_flat_variants(torch, g, steps, warmup, seed):
    """The decode shape of the flat workload (16 x 16384 x 7168) in the other scale modes and in MXFP4, and with 32
    and 64 activation rows (one pass over the weights for all of them), each with rotating copies of the pre-shuffled
    weights (larger than the Infinity Cache together), priced against HBM."""
    import ctypes
    n, k = 16384, 7168
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    xa64 = torch.randn((64, k), generator=gen, device="cuda")
    xb = torch.randn((n, k), generator=gen, device="cuda")
    L = g.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = []
    for name, fp4, m in (("flatmm_mx_tiled", False, 16), ("flatmm_block", False, 16), ("flatmm_mxfp4", True, 16),
                         ("flatmm_rowcol", False, 32), ("flatmm_rowcol", False, 64), ("flatmm_mx_tiled", False, 64),
                         ("gemm_blockscale_row_major_b", False, 16), ("gemm_blockscale_row_major_b", False, 64)):
        xa = xa64[:m].contiguous()
        c = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        shuffled = 1
        if name == "gemm_blockscale_row_major_b":
            # the reference's own entry point and operand layout at decode sizes: routed to the flat kernel, which
            # stages the row-major weight rows through LDS
            (a, sfa), (b, sfb) = g.quantize(xa, g.BLOCK, 1), g.quantize(xb, g.BLOCK, 128)
            mode, entry, wbytes, sbytes = g.BLOCK, L.a8w8_gemm_blockscale, n * k, 4 * (n // 128) * (k // 128) + 4 * m * (k // 128)
            shuffled = 0
        elif name == "flatmm_rowcol":
            (a, sfa), (b, sfb) = g.quantize(xa, g.ROWCOL), g.quantize(xb, g.ROWCOL)
            mode, entry, wbytes, sbytes = g.ROWCOL, L.a8w8_flatmm, n * k, 4 * (n + m)
        elif fp4:
            (a, sfa), (b, sfb) = g.quantize_mxfp4(xa, tiled=True), g.quantize_mxfp4(xb, tiled=True)
            mode, entry, wbytes, sbytes = g.MX_TILED, L.a4w4_flatmm, n * k // 2, n * k // 32 + m * k // 32
        elif name == "flatmm_mx_tiled":
            (a, sfa), (b, sfb) = g.quantize(xa, g.MX_TILED), g.quantize(xb, g.MX_TILED)
            mode, entry, wbytes, sbytes = g.MX_TILED, L.a8w8_flatmm, n * k, n * k // 32 + m * k // 32
        else:
            (a, sfa), (b, sfb) = g.quantize(xa, g.BLOCK, 1), g.quantize(xb, g.BLOCK, 128)
            mode, entry, wbytes, sbytes = g.BLOCK, L.a8w8_flatmm, n * k, 4 * (n // 128) * (k // 128) + 4 * m * (k // 128)
        bs = g.preshuffle_b_device(b) if shuffled else b
        copies = [bs] + [bs.clone() for _ in range(3 if not fp4 else 7)]
        args = [g.raw_gemm_args(a.data_ptr(), x.data_ptr(), c.data_ptr(), sfa.data_ptr(), sfb.data_ptr(), m, n, k, mode, g.BF16,
                                b_preshuffled=shuffled) for x in copies]
        kernel = "flatmm_a8w8 (FP4 mode)" if fp4 else g.kernel_name(args[0])
        refs = [ctypes.byref(x) for x in args]
        mask = len(copies) - 1

        def fn(i, entry=entry, refs=refs, mask=mask):
            if entry(refs[i & mask], stream) != 0:
                raise RuntimeError("flat call failed")

        ms, wall = time_best_of(torch, fn, steps, warmup)
        abytes = wbytes + sbytes + a.numel() + 2 * m * n
        out.append({"workload": f"{name}_{m}x{n}x{k}", "m": m, "n": n, "k": k, "kernel": kernel,
                    "ms_per_launch": ms, "wall_ms_per_launch": wall, "algorithmic_bytes": abytes, "gbs": abytes / ms / 1e6,
                    "frac_hbm_peak": abytes / ms / 1e6 / PEAK_HBM_GBS,
                    "note": f"{len(copies)} rotating copies of the weights ({len(copies) * wbytes // 10**6} MB)"})
        del copies, args, refs, bs, a, b, sfa, sfb
        torch.cuda.empty_cache()
    return out


def cpu_baseline(name, inp, c_gpu, torch, budget_s=15.0, max_rows=256):
    """Times the oracle (port of the reference's host GEMM: per-MAC software fp8 decode,
    OpenMP over (i, j), gemm_a8w8_blockscale_host.cc:66-90) on the first rows of the same
    problem -- as many as about budget_s seconds allow, at most max_rows -- and checks the GPU
    result on that slab.  A slab smaller than the problem is extrapolated linearly and says so."""
    import numpy as np
    import oracle
    mode, m, n, k, _ = WORKLOADS[name]
    a = inp["a"].cpu().numpy()
    b = inp["b"].cpu().numpy()
    sfa = inp["sfa"].cpu().numpy()
    sfb = inp["sfb"].cpu().numpy()
    omode = {"mx": oracle.MX, "rowcol": oracle.ROWCOL, "block": oracle.BLOCK, "tensor": oracle.TENSOR,
             "flat": oracle.ROWCOL}[mode]
    t0 = time.perf_counter()
    oracle.gemm_ref(a, b, sfa, sfb, omode, rows=(0, 1), decode_per_mac=True)
    t_row = time.perf_counter() - t0
    rows = int(max(1, min(m, max_rows, budget_s / max(t_row, 1e-4))))
    t0 = time.perf_counter()
    ref = oracle.gemm_ref(a, b, sfa, sfb, omode, rows=(0, rows), decode_per_mac=True)
    dt = time.perf_counter() - t0
    got = c_gpu[:rows].float().cpu().numpy()
    ok = np.abs(got - ref) <= 1e-2 * np.abs(ref) + 1e-2
    whole = rows == m
    sample = (f"the whole problem ({m} rows of C), {dt:.2f} s" if whole else
              f"first {rows} of {m} rows of C (all N, all K), {dt:.2f} s; full problem extrapolates linearly to {dt * m / rows:.0f} s")
    return {
        "value": 2.0 * rows * n * k / dt / 1e12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
        "sample": sample, "extrapolated": not whole, "gpu_slab_within_tolerance": float(ok.mean()),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="mxfp8_8192", choices=sorted(w for w in WORKLOADS if WORKLOADS[w][0] not in ("bf16", "f4")))
    ap.add_argument("--seed", type=int, default=0xA8A80004)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="time only the selected workload")
    ap.add_argument("--operands", default="as_configured", choices=["as_configured", "zeros", "random_bytes"],
                    help="measurement aid: replace the selected workload's quantised operands (the result is then not the configuration's)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1")

    import torch
    import gcnasm_amd as g
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    g.lib()     # raises if the HIP library has not been built; there is no fallback path
    torch.cuda.set_device(0)

    res, inp, c = run_workload(args.workload, torch, g, args.steps, args.warmup, args.seed, operands=args.operands)
    mode, m, n, k, abytes = WORKLOADS[args.workload]
    if mode == "flat":
        value, unit = res["gbs"], "GB/s"
        roof = {"bound": "hbm", "achieved": res["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": res["gbs"] / PEAK_HBM_GBS, "traffic": measured_traffic().get(args.workload), "kernel": "flatmm_a8w8"}
    else:
        value, unit = res["tflops"], "TFLOP/s"
        # the dominant kernel alone (for MX: the GEMM launch without the two scale re-ordering launches)
        kern_tflops = res.get("tflops_gemm_kernel", res["tflops"])
        roof = {"bound": "mfma", "achieved": kern_tflops, "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                "frac": kern_tflops / PEAK_FP8_TFLOPS, "traffic": measured_traffic().get(args.workload),
                "kernel": res.get("kernel")}
    line = {
        "metric": METRIC, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": res["ms_per_launch"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3", "data": "synthetic",
        "config": {"workload": args.workload, "m": m, "n": n, "k": k, "out": "bf16", "accumulate": "fp32",
                   "algorithmic_bytes": abytes, "flop": 2 * m * n * k},
        "roofline": roof,
    }
    if args.operands != "as_configured" or g.lib().a8w8_version() < 0 or os.environ.get("MI355_A8W8_LIBRARY"):
        # a measurement run: other operand contents, or a library built with measurement switches
        line["config"]["measurement_run"] = {"operands": args.operands, "library": g.library_path(),
                                             "library_version": g.lib().a8w8_version()}
    for key in ("step", "ms_gemm_kernel", "tflops_gemm_kernel", "ms_row_major_scales_one_launch",
                "tflops_row_major_scales_one_launch", "first_region_ms_per_step", "first_region_tflops"):
        if key in res:
            line["config"][key] = res[key]
    line["config"]["timing"] = (f"{CONDITION_S} s of the same launches (counted in neither W nor K) bring the clocks to what the chip "
                                "sustains, then W warm-up and K timed launches between two HIP events on the launch stream; "
                                "first_region_* is the same W + K protocol run before that on the chip as found")
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(args.workload, inp, c, torch)
    del inp, c
    torch.cuda.empty_cache()
    if not args.no_extra:
        others = []
        for name in WORKLOADS:
            if name == args.workload or name in SELECT_ONLY:
                continue
            r, i2, c2 = run_workload(name, torch, g, args.steps, args.warmup, args.seed + 1, headline=False)
            r["timing"] = "best of 3 regions of K launches after 100 ms of warm-up"
            if not args.no_cpu and WORKLOADS[name][0] not in ("bf16", "f4"):
                # the two small configurations whole, the large ones on a 64-row slab
                r["cpu_baseline"] = cpu_baseline(name, i2, c2, torch, budget_s=4.0, max_rows=WORKLOADS[name][1] if WORKLOADS[name][1] <= 256 else 64)
            others.append(r)
            del i2, c2
            torch.cuda.empty_cache()
        others.extend(run_quantizers(torch, g, args.steps, args.warmup, args.seed + 2))
        others.extend(run_reference_program_sizes(torch, g, args.steps, args.warmup, args.seed + 3))
        others.extend(run_flat_variants(torch, g, args.steps, args.warmup, args.seed + 4))
        line["other_workloads"] = others
        # the secondary results in short form inside `config`, which a truncated record still holds
        by_name = {w["workload"]: w for w in others}
        def pick(workload, key):
            v = by_name.get(workload, {}).get(key)
            return None if v is None else round(v, 4)
        line["config"].update(
            c2_frac=pick("rowcol_4096", "frac_fp8_peak"), c3_frac=pick("block_4096x7168x2048", "frac_fp8_peak"),
            c3_us=pick("block_4096x7168x2048", "ms_per_launch") and round(by_name["block_4096x7168x2048"]["ms_per_launch"] * 1e3, 2),
            c5_frac_hbm=pick("flatmm_16x16384x7168", "frac_hbm_peak"), c5_frac_hbm_in_graph=pick("flatmm_16x16384x7168", "frac_hbm_peak_in_graph"),
            c5_frac_of_achievable_read=pick("flatmm_16x16384x7168", "frac_of_achievable_read"),
            block_fp32_4096_vs_ref=pick("block_fp32_4096", "vs_reference_published"),
            block_fp32_8192_vs_ref=pick("block_fp32_8192", "vs_reference_published"),
            block_fp32_16384_vs_ref=pick("block_fp32_16384", "vs_reference_published"),
            gemm_rowcol_256x8192x8192_us=pick("gemm_rowcol_256x8192x8192", "ms_per_launch") and round(by_name["gemm_rowcol_256x8192x8192"]["ms_per_launch"] * 1e3, 2),
            flatmm_rowcol_64_frac_hbm=pick("flatmm_rowcol_64x16384x7168", "frac_hbm_peak"),
            a16w16_4096_frac=pick("a16w16_4096", "frac_bf16_peak"), mxfp4_8192_frac=pick("mxfp4_8192", "frac_fp4_peak"))
    print(json.dumps(line))


if __name__ == "__main__":
    main()
