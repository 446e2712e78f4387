"""gcnasm_amd -- MI355X (gfx950) A8W8 FP8 GEMM library: Python binding of libmi355a8w8.so.

The compute lives in hand-written HIP kernels behind a C ABI (include/mi355_a8w8.h); this
package only loads that library and passes device pointers to it.  There is no fallback:
if the library is missing or the GPU is not gfx950 the calls raise.
"""
from .api import (  # noqa: F401
    A8W8Error, BF16, BLOCK, FNUZ, FP32, MX, MX_TILED, OCP, ROWCOL, TENSOR, GemmArgs, build_library, cvt_e4m3_to_f32,
    cvt_f32_to_e4m3, flatmm, flatmm_a16w16, flatmm_a4w4, gemm, gemm_a16w16, gemm_a4w4, init, quantize_mxfp4, gemm_blockscale, kernel_name, lib, library_path, load_weights, save_weights, mx_tile_scales, mx_tile_scales_ab, mx_tiled_bytes, preshuffle_b, preshuffle_b_bf16_device,
    preshuffle_b_device, quantize, raw_gemm_args, status_string, unshuffle_b,
)
from .ops import register as register_torch_ops  # noqa: E402,F401
