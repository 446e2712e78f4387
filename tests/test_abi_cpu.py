"""Host-side checks of the C ABI that need no GPU: the library loads, exports every symbol
the header declares, and rejects bad arguments with the documented status codes (argument
validation runs before any device call, mirroring the reference harness's rejects at
opus_gemm/block_scale_gemm/gemm_a8w8_blockscale_host.cc:175-187)."""
import ctypes
import os
import re

import numpy as np
import pytest

import gcnasm_amd as g

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_declared_symbol_is_exported():
    text = open(os.path.join(ROOT, "include", "mi355_a8w8.h")).read()
    names = set(re.findall(r"A8W8_API\s+[\w\s\*]+?\b(a8w8_\w+)\s*\(", text))
    assert {"a8w8_gemm", "a8w8_gemm_blockscale", "a8w8_flatmm", "a8w8_preshuffle_b", "a8w8_cvt_f32_to_e4m3",
            "a8w8_cvt_e4m3_to_f32", "a8w8_status_string", "a8w8_init"} <= names
    L = ctypes.CDLL(g.library_path())
    for n in names:
        assert hasattr(L, n), n


def _ok_args(mode=g.BLOCK, m=256, n=256, k=256, **kw):
    # device addresses are never dereferenced on the host; any aligned non-null value will do
    return g.raw_gemm_args(0x1000, 0x2000, 0x3000, 0x4000, 0x5000, m, n, k, mode, **kw)


@pytest.mark.parametrize("mutate,want", [
    (lambda a: setattr(a, "a", None), -1),
    (lambda a: setattr(a, "sfb", None), -1),
    (lambda a: setattr(a, "m", 0), -2),
    (lambda a: setattr(a, "batch", -1), -2),
    (lambda a: setattr(a, "n", 200), -3),          # N % 128 for block scales
    (lambda a: setattr(a, "k", 192), -3),          # K % 128 for block scales
    (lambda a: setattr(a, "stride_a", 128), -4),
    (lambda a: setattr(a, "stride_c", 100), -4),
    (lambda a: setattr(a, "stride_sfa", 8), -4),
    (lambda a: setattr(a, "scale_mode", 7), -6),
    (lambda a: setattr(a, "c_dtype", 3), -6),
])
def test_gemm_rejects_bad_arguments(mutate, want):
    a = _ok_args()
    mutate(a)
    assert g.lib().a8w8_gemm(ctypes.byref(a), None) == want
    assert g.kernel_name(a) is None
    assert g.status_string(want) != "unknown status"


def test_c_stride_limit_applies_to_the_256_tile_kernels_only():
    """The two 256-tile kernels address a C tile's 256 rows with unsigned 32-bit byte offsets:
    (255 stride_c + 256) * sizeof(element) < 2^32.  Rejected before any device call; every other kernel takes any stride."""
    L, ref = g.lib(), ctypes.byref
    fp32_max, bf16_max = 4_210_751, 8_421_503
    for mode, k in [(g.ROWCOL, 512), (g.BLOCK, 512), (g.ROWCOL, 384)]:          # wide, persist, persist (odd step count)
        for c_dtype, most in [(g.FP32, fp32_max), (g.BF16, bf16_max)]:
            big = _ok_args(mode=mode, m=4096, n=4096, k=k, c_dtype=c_dtype, stride_c=most + 1)
            assert g.kernel_name(_ok_args(mode=mode, m=4096, n=4096, k=k, c_dtype=c_dtype)) in ("gemm_a8w8_wide", "gemm_a8w8_persist")
            assert L.a8w8_gemm(ref(big), None) == -7
            fits = _ok_args(mode=mode, m=4096, n=4096, k=k, c_dtype=c_dtype, stride_c=most)
            assert L.a8w8_gemm(ref(fits), None) != -7
    # the 128-tile kernel, the one-thread-per-element kernel and the flat kernel use 64-bit pointers
    for kw in [dict(mode=g.ROWCOL, m=256, n=256, k=256), dict(mode=g.ROWCOL, m=4096, n=4096, k=200, stride_a=200, stride_b=200),
               dict(mode=g.ROWCOL, m=16, n=4096, k=4096)]:
        a = _ok_args(stride_c=1 << 24, **kw)
        assert g.kernel_name(a) in ("gemm_a8w8_tile128", "gemm_a8w8_general", "flatmm_a8w8")
        assert L.a8w8_gemm(ref(a), None) != -7
    # siblings: m, n, k in their own elements
    big = _ok_args(mode=g.TENSOR, m=4096, n=4096, k=512, c_dtype=g.FP32, stride_c=fp32_max + 1)
    assert L.a16w16_gemm(ref(big), None) == -7
    small = _ok_args(mode=g.TENSOR, m=256, n=256, k=256, c_dtype=g.FP32, stride_c=fp32_max + 1)
    assert L.a16w16_gemm(ref(small), None) != -7
    big = _ok_args(mode=g.MX_TILED, m=4096, n=4096, k=1024, c_dtype=g.FP32, stride_c=fp32_max + 1)
    assert L.a4w4_gemm(ref(big), None) == -7
    small = _ok_args(mode=g.MX_TILED, m=64, n=64, k=256, c_dtype=g.FP32, stride_c=fp32_max + 1)
    assert L.a4w4_gemm(ref(small), None) != -7


def test_null_struct_and_mx_group():
    assert g.lib().a8w8_gemm(None, None) == -1
    assert g.lib().a8w8_gemm_blockscale(None, None) == -1
    a = _ok_args(mode=g.MX, k=48)
    assert g.lib().a8w8_gemm(ctypes.byref(a), None) == -3
    a = _ok_args(mode=g.ROWCOL, m=70000, k=32768, n=16)     # 2.29e9 bytes of A
    assert g.lib().a8w8_gemm(ctypes.byref(a), None) == -7


def test_flatmm_preconditions():
    a = _ok_args(mode=g.ROWCOL, m=16, n=256, k=256, b_preshuffled=1)
    assert g.kernel_name(a) == "flatmm_a8w8"
    for mutate, want in [(lambda x: setattr(x, "b_preshuffled", 0), -6), (lambda x: setattr(x, "scale_mode", g.MX), -6),
                         (lambda x: setattr(x, "m", 129), -2), (lambda x: setattr(x, "n", 250), -3),
                         (lambda x: setattr(x, "k", 96), -3), (lambda x: setattr(x, "a", 0x1001), -5)]:
        b = _ok_args(mode=g.ROWCOL, m=16, n=256, k=256, b_preshuffled=1)
        mutate(b)
        if b.k == 96:
            b.stride_a = 96
        assert g.lib().a8w8_flatmm(ctypes.byref(b), None) == want


def test_gemm_on_shuffled_weights_preconditions():
    """a8w8_gemm reads B in the flat GEMM's layout too: whole 16-row groups and 128-wide K steps, aligned pointers."""
    L = g.lib()
    ok = _ok_args(mode=g.ROWCOL, m=4096, n=4096, k=512, b_preshuffled=1)
    ok.stride_b = 0                                           # not read for shuffled weights
    assert g.kernel_name(ok) == "gemm_a8w8_wide"
    assert g.kernel_name(_ok_args(mode=g.BLOCK, m=300, n=512, k=512, b_preshuffled=1)) == "gemm_a8w8_tile128"
    assert g.kernel_name(_ok_args(mode=g.ROWCOL, m=16, n=256, k=256, b_preshuffled=1)) == "flatmm_a8w8"     # flat when it can
    # row-major weights, at most 128 rows: the flat kernel where it can run and the model calls it faster
    rm = dict(mode=g.ROWCOL, n=16384, k=7168)
    assert g.kernel_name(_ok_args(m=64, **rm)) == "flatmm_a8w8"
    assert g.kernel_name(_ok_args(m=128, mode=g.ROWCOL, n=16384, k=8192)) == "gemm_a8w8_tile128"       # two passes, rows 8192 apart
    assert g.kernel_name(_ok_args(m=129, **rm)) == "gemm_a8w8_tile128"
    assert g.kernel_name(_ok_args(m=64, mode=g.ROWCOL, n=16384 + 8, k=7168)) == "gemm_a8w8_tile128"      # n % 16 != 0
    assert g.kernel_name(_ok_args(m=16, mode=g.MX, n=4096, k=4096)) == "gemm_a8w8_tile128"              # row-major MX scales
    assert g.kernel_name(_ok_args(m=16, mode=g.BLOCK, n=4096, k=4096)) == "flatmm_a8w8"
    # skinny problems: the side a cost model of the two kernels calls faster (the measured winners)
    big = dict(n=16384, k=7168, b_preshuffled=1)
    assert g.kernel_name(_ok_args(m=64, mode=g.ROWCOL, **big)) == "flatmm_a8w8"
    assert g.kernel_name(_ok_args(m=64, mode=g.MX_TILED, **big)) == "flatmm_a8w8"
    wide = dict(n=28672, k=4096, b_preshuffled=1)                # 224 workgroups on the 128-tile kernel, short rows
    assert g.kernel_name(_ok_args(m=48, mode=g.ROWCOL, **wide)) == "flatmm_a8w8"
    assert g.kernel_name(_ok_args(m=96, mode=g.ROWCOL, **wide)) == "gemm_a8w8_tile128"       # (at 64 rows the two are level)
    assert g.kernel_name(_ok_args(m=48, mode=g.MX_TILED, **wide)) == "flatmm_a8w8"
    assert g.kernel_name(_ok_args(m=64, mode=g.MX_TILED, **wide)) == "gemm_a8w8_tile128"
    # past 64 rows the flat kernel makes two passes over weights of this size: the 128-tile kernel's 128 x 64 tiles win
    assert g.kernel_name(_ok_args(m=96, mode=g.ROWCOL, **big)) == "gemm_a8w8_tile128"
    assert g.kernel_name(_ok_args(m=128, mode=g.MX_TILED, **big)) == "gemm_a8w8_tile128"
    assert g.kernel_name(_ok_args(m=64, n=4096, k=4096, mode=g.ROWCOL, b_preshuffled=1)) == "flatmm_a8w8"
    assert g.kernel_name(_ok_args(m=64, n=16384, k=7104, mode=g.ROWCOL, b_preshuffled=1)) == "flatmm_a8w8"   # K % 128 != 0: flat only
    for mutate, want in [(lambda x: setattr(x, "n", 4088), -3), (lambda x: setattr(x, "k", 448), -3),
                         (lambda x: setattr(x, "b", 0x2008), -5), (lambda x: setattr(x, "stride_a", 520), -5)]:
        b = _ok_args(mode=g.ROWCOL, m=4096, n=4096, k=512, b_preshuffled=1)
        mutate(b)
        assert L.a8w8_gemm(ctypes.byref(b), None) == want, want
        assert g.kernel_name(b) is None


def test_kernel_selection():
    big = dict(m=4096, n=4096)                       # 256 tiles of 256 x 256: enough for every compute unit
    assert g.kernel_name(_ok_args(**big)) == "gemm_a8w8_persist"
    assert g.kernel_name(_ok_args(mode=g.MX, **big)) == "gemm_a8w8_persist"
    # per-tensor, row/col and tiled-MX scales with an even number of K steps: the four-wave kernel
    assert g.kernel_name(_ok_args(mode=g.ROWCOL, **big)) == "gemm_a8w8_wide"
    assert g.kernel_name(_ok_args(mode=g.TENSOR, k=1024, **big)) == "gemm_a8w8_wide"
    assert g.kernel_name(_ok_args(mode=g.ROWCOL, k=384, **big)) == "gemm_a8w8_persist"
    # a single K step: the 128-tile kernel at any size (the pipelined kernels stage two steps ahead)
    assert g.kernel_name(_ok_args(mode=g.ROWCOL, k=128, **big)) == "gemm_a8w8_tile128"
    # row strides of 2^23 bytes and more keep their kernel (row offsets are full 32-bit products)
    assert g.kernel_name(_ok_args(mode=g.ROWCOL, m=512, n=16, k=256, stride_b=1 << 23)) == "gemm_a8w8_tile128"
    assert g.lib().a8w8_gemm(ctypes.byref(_ok_args(mode=g.ROWCOL, m=4096, n=512, k=256, stride_b=1 << 23)), None) == -7   # 2 GiB span
    # every scale mode: 128 x 128 tiles while all of them fit on the chip at once (two workgroups per compute unit)
    assert g.kernel_name(_ok_args()) == "gemm_a8w8_tile128"
    assert g.kernel_name(_ok_args(mode=g.ROWCOL, m=1024, n=2048, k=128)) == "gemm_a8w8_tile128"
    for mode in (g.TENSOR, g.ROWCOL, g.BLOCK, g.MX, g.MX_TILED):
        assert g.kernel_name(_ok_args(mode=mode, m=2048, n=4096)) == "gemm_a8w8_tile128"       # 512 workgroups
        assert g.kernel_name(_ok_args(mode=mode, m=2049, n=4096)) != "gemm_a8w8_tile128"       # 544
        assert g.kernel_name(_ok_args(mode=mode, m=1024, n=1024, batch=8)) == "gemm_a8w8_tile128"
        assert g.kernel_name(_ok_args(mode=mode, m=1024, n=1024, batch=9)) != "gemm_a8w8_tile128"
    assert g.kernel_name(_ok_args(mode=g.TENSOR, m=2304, n=4096)) == "gemm_a8w8_wide"
    assert g.kernel_name(_ok_args(m=2304, n=4096)) == "gemm_a8w8_persist"
    assert g.kernel_name(_ok_args(mode=g.ROWCOL, k=200)) == "gemm_a8w8_general"
    a = _ok_args(mode=g.ROWCOL)
    a.a = 0x1004
    assert g.kernel_name(a) == "gemm_a8w8_general"


def test_tiled_mx_mode_selection_and_reorder_preconditions():
    big = dict(m=4096, n=4096)
    assert g.kernel_name(_ok_args(mode=g.MX_TILED, **big)) == "gemm_a8w8_wide"
    # an odd number of K steps: the 128-tile kernel whatever the size (the four-wave kernel walks K in pairs)
    assert g.kernel_name(_ok_args(mode=g.MX_TILED, k=384, **big)) == "gemm_a8w8_tile128"
    assert g.kernel_name(_ok_args(mode=g.MX_TILED, k=128, **big)) == "gemm_a8w8_tile128"
    assert g.kernel_name(_ok_args(mode=g.MX_TILED, k=384)) == "gemm_a8w8_tile128"
    assert g.kernel_name(_ok_args(mode=g.MX_TILED, k=352, stride_a=352, stride_b=352)) == "gemm_a8w8_general"
    a = _ok_args(mode=g.MX_TILED, k=48)
    assert g.lib().a8w8_gemm(ctypes.byref(a), None) == -3
    a = _ok_args(mode=g.MX_TILED)
    a.sfa = 0x4004                                                                      # tiled scales need 16-byte alignment
    assert g.kernel_name(a) == "gemm_a8w8_general"
    L = g.lib()
    assert L.a8w8_mx_tiled_bytes(64, 512) == 1024 and L.a8w8_mx_tiled_bytes(65, 513) == 4096
    assert L.a8w8_mx_tiled_bytes(0, 512) == 0
    assert g.mx_tiled_bytes(8192, 8192) == 8192 * 256 == L.a8w8_mx_tiled_bytes(8192, 8192)
    assert L.a8w8_mx_tile_scales(None, 64, 512, 16, 0x1000, None) == -1
    assert L.a8w8_mx_tile_scales(0x1000, 0, 512, 16, 0x2000, None) == -2
    assert L.a8w8_mx_tile_scales(0x1000, 64, 500, 16, 0x2000, None) == -3
    assert L.a8w8_mx_tile_scales(0x1000, 64, 512, 8, 0x2000, None) == -4
    assert L.a8w8_mx_tile_scales(0x1000, 64, 512, 16, 0x2004, None) == -5
    assert L.a8w8_mx_tile_scales_ab(0x1000, 64, 16, 0x2000, None, 64, 16, 0x3000, 512, None) == -1
    assert L.a8w8_mx_tile_scales_ab(0x1000, 64, 16, 0x2000, 0x4000, 64, 8, 0x3000, 512, None) == -4


def test_pipelined_kernels_use_no_scratch():
    """The build keeps the compiler's per-kernel resource report.  A register spilled inside the K loop
    of the persistent GEMM is reloaded behind a wait for every direct-to-LDS load in flight (the reload
    and the loads share one in-order counter), which costs tens of percent: none may spill."""
    path = os.path.join(ROOT, "gcnasm_amd", "libmi355a8w8.resources.txt")
    if not os.path.exists(path):
        pytest.skip("resource report not written by this build of the library")
    text = open(path).read()
    blocks = text.split("Function Name: ")[1:]
    seen = 0
    for b in blocks:
        name = b.split()[0]
        if "gemm_a8w8_persist" in name or "gemm_a8w8_wide" in name or "gemm_a8w8_tile128" in name or "flatmm_a8w8" in name:
            seen += 1
            scratch = int(re.search(r"ScratchSize \[bytes/lane\]: (\d+)", b).group(1))
            assert scratch == 0, (name, scratch)
    assert seen >= 40
    # the four-wave kernels name their accumulator registers themselves: the build checks that the
    # compiler put nothing of its own there (gcnasm_amd/csrc/check_isa.py) and records the verdict
    assert "accumulator registers untouched by the compiler" in text
    # ... and that every 16-byte buffer store of a C tile is followed by the idle cycles its data registers need
    assert re.search(r"16-byte buffer stores: \d+ checked, none with a write to its data registers in the two slots behind it", text)
    # MXFP8 flat GEMM: four weight tiles x four row groups exists (and is among the kernels checked above)
    assert "flatmm_a8w8ILi4ELi4ELi0ELi4ELb0EE" in text


def test_sibling_entry_points_reject_bad_arguments():
    """bf16, MXFP4, quantiser and conversion entry points: every reject happens before any device call."""
    L = g.lib()
    ref = ctypes.byref
    # a16w16_gemm: strides in bf16 elements
    a = _ok_args(mode=g.TENSOR)
    for mutate, want in [(lambda x: setattr(x, "c", None), -1), (lambda x: setattr(x, "k", 0), -2),
                         (lambda x: setattr(x, "c_dtype", 7), -6),
                         (lambda x: setattr(x, "stride_b", 100), -4)]:
        b = _ok_args(mode=g.TENSOR)
        mutate(b)
        assert L.a16w16_gemm(ref(b), None) == want
    assert L.a16w16_gemm(None, None) == -1
    # a16w16_flatmm
    for mutate, want in [(lambda x: setattr(x, "b_preshuffled", 0), -6), (lambda x: setattr(x, "m", 129), -2),
                         (lambda x: setattr(x, "n", 250), -3), (lambda x: setattr(x, "k", 48), -3),
                         (lambda x: setattr(x, "stride_a", 260), -5), (lambda x: setattr(x, "a", 0x1008), -5)]:
        b = _ok_args(mode=g.TENSOR, m=16, n=256, k=256, b_preshuffled=1)
        mutate(b)
        assert L.a16w16_flatmm(ref(b), None) == want, want
    # a4w4_gemm: m, n, k and strides in E2M1 elements
    for mutate, want in [(lambda x: setattr(x, "sfa", None), -1), (lambda x: setattr(x, "scale_mode", g.ROWCOL), -6),
                         (lambda x: setattr(x, "k", 48), -3), (lambda x: setattr(x, "stride_a", 200), -4),
                         (lambda x: setattr(x, "stride_a", 259), -5),       # rows must start on a byte
                         (lambda x: setattr(x, "stride_sfa", 4), -4)]:
        b = _ok_args(mode=g.MX, m=64, n=64, k=256)
        mutate(b)
        assert L.a4w4_gemm(ref(b), None) == want, want
    # a4w4_flatmm: pre-shuffled packed weights, tiled scales only
    for mutate, want in [(lambda x: setattr(x, "b_preshuffled", 0), -6), (lambda x: setattr(x, "scale_mode", g.MX), -6),
                         (lambda x: setattr(x, "m", 129), -2), (lambda x: setattr(x, "n", 250), -3),
                         (lambda x: setattr(x, "k", 192), -3), (lambda x: setattr(x, "stride_a", 272), -5),
                         (lambda x: setattr(x, "sfb", 0x5004), -5), (lambda x: setattr(x, "sfa", None), -1)]:
        b = _ok_args(mode=g.MX_TILED, m=16, n=256, k=256, b_preshuffled=1)
        mutate(b)
        assert L.a4w4_flatmm(ref(b), None) == want, want
    # quantisers
    assert L.a8w8_quantize(None, 4, 32, 32, 0x2000, 0x3000, g.ROWCOL, 1, None) == -1
    assert L.a8w8_quantize(0x1000, 0, 32, 32, 0x2000, 0x3000, g.ROWCOL, 1, None) == -2
    assert L.a8w8_quantize(0x1000, 4, 32, 16, 0x2000, 0x3000, g.ROWCOL, 1, None) == -4
    assert L.a8w8_quantize(0x1000, 4, 100, 100, 0x2000, 0x3000, g.BLOCK, 1, None) == -3
    assert L.a8w8_quantize(0x1000, 100, 128, 128, 0x2000, 0x3000, g.BLOCK, 128, None) == -3
    assert L.a8w8_quantize(0x1000, 4, 48, 48, 0x2000, 0x3000, g.MX, 1, None) == -3
    assert L.a8w8_quantize(0x1000, 4, 32, 32, 0x2000, 0x3000, 9, 1, None) == -6
    assert L.a4w4_quantize_mx(0x1000, 4, 48, 48, 0x2000, 0x3000, 0, None) == -3
    assert L.a4w4_quantize_mx(0x1000, 4, 64, 32, 0x2000, 0x3000, 0, None) == -4
    assert L.a4w4_quantize_mx(0x1000, 4, 64, 64, 0x2000, 0x3002, 1, None) == -5
    # conversions return a status like every other entry point; zero elements is a no-op, not an error
    assert L.a8w8_cvt_f32_to_e4m3(None, 0x2000, 16, g.OCP, 0, None) == -1
    assert L.a8w8_cvt_f32_to_e4m3(0x1000, 0x2000, 16, 5, 0, None) == -6
    assert L.a8w8_cvt_e4m3_to_f32(0x1000, None, 16, g.OCP, None) == -1
    assert L.a8w8_cvt_e4m3_to_f32(0x1000, 0x2000, 16, 2, None) == -6
    assert L.a8w8_cvt_f32_to_e4m3(None, None, 0, g.OCP, 0, None) == 0
    assert L.a8w8_cvt_e4m3_to_f32(None, None, 0, g.FNUZ, None) == 0
    # block scales: the A-side scale offsets of all K groups have to fit 32 bits
    assert L.a8w8_gemm(ctypes.byref(_ok_args(mode=g.BLOCK, m=256, n=256, k=1024, stride_sfa=1 << 27)), None) == -7
    assert L.a8w8_preshuffle_b_device(0x1000, 0x2000, 40, 192, None) == -3
    assert L.a8w8_preshuffle_b_device(0x1000, 0x2004, 48, 192, None) == -5


def test_good_arguments_pass_validation_and_stop_at_the_device():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present: the call would launch")
    assert g.lib().a8w8_gemm(ctypes.byref(_ok_args()), None) == -9
    assert "gfx950" in g.status_string(-9)


def test_header_states_the_tiled_scale_layout(orc):
    """The byte position include/mi355_a8w8.h gives for the exponent of (row r, 32-block kb) in the MX_TILED layout,
    evaluated as written, is where the oracle's layout walk puts it (ragged row and K counts included)."""
    text = open(os.path.join(ROOT, "include", "mi355_a8w8.h")).read()
    m = re.search(r"the exponent of \(row r, block kb\) is byte\s*\*\s*(.+?)\n\s*\*\s*(.+?)\n\s*\*\s*\(pair =", text, re.S)
    assert m, "the header no longer states the formula in the expected place"
    formula = (m.group(1) + " " + m.group(2)).replace("ceil(rows/64)", "((rows + 63) // 64)")
    formula = re.sub(r"(?<![/])/(?![/])", "//", formula)
    size = re.search(r"ceil\(k/512\) \* ceil\(rows/64\) \* 1024 bytes", text)
    assert size, "the header no longer states the size"
    for rows, k in ((64, 512), (200, 1600), (130, 96), (1, 32)):
        kb_n = k // 32
        rng = np.random.Generator(np.random.Philox(rows))
        sf = rng.integers(0, 255, (rows, kb_n)).astype(np.uint8)
        tiled = orc.mx_tile_scales(sf)
        assert tiled.size == ((k + 511) // 512) * ((rows + 63) // 64) * 1024 == g.lib().a8w8_mx_tiled_bytes(rows, k)
        seen = np.zeros(tiled.size, bool)
        for r in range(rows):
            rr = r % 64
            for kb in range(kb_n):
                pos = eval(formula, {"rows": rows, "r": r, "rr": rr, "kb": kb})
                assert tiled[pos] == sf[r, kb], (rows, k, r, kb, pos)
                seen[pos] = True
        assert (tiled[~seen] == 127).all()


def test_host_preshuffle_matches_oracle(orc):
    rng = np.random.Generator(np.random.Philox(1))
    b = rng.integers(0, 256, (48, 192)).astype(np.uint8)
    bs = g.preshuffle_b(b)
    assert (bs == orc.preshuffle_b(b)).all()
    assert (g.unshuffle_b(bs, 48, 192) == b).all()
    assert g.lib().a8w8_preshuffle_b(b.ctypes.data, bs.ctypes.data, 40, 192) == -3


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    import gcnasm_amd.api as api
    monkeypatch.setattr(api, "_lib", None)
    monkeypatch.setattr(api, "_SO", str(tmp_path / "nope.so"))
    with pytest.raises(FileNotFoundError):
        api.lib()
