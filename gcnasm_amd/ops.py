"""torch operator wrappers over the C ABI (the style of the reference's FFI registrations,
mla_agentic_v0/csrc/tvm_api.cc:5-33, with torch.library in place of TVM-FFI).

`register()` defines, once per process,

    torch.ops.mi355_a8w8.gemm(a, b, sfa, sfb, scale_mode, out_fp32)     -> C      (a8w8_gemm)
    torch.ops.mi355_a8w8.flatmm(a, b_shuffled, sfa, sfb, n, scale_mode, out_fp32) (a8w8_flatmm)
    torch.ops.mi355_a8w8.gemm_a16w16(a, b, out_fp32)                              (a16w16_gemm)
    torch.ops.mi355_a8w8.quantize(x, scale_mode, group_rows) -> (q, scales)       (a8w8_quantize)
    torch.ops.mi355_a8w8.quantize_mxfp4(x, tiled) -> (q, scales)                  (a4w4_quantize_mx)
    torch.ops.mi355_a8w8.gemm_a4w4(a, b, sfa, sfb, scale_mode, out_fp32)          (a4w4_gemm)
    torch.ops.mi355_a8w8.flatmm_a4w4(a, b_shuffled, sfa, sfb, n, out_fp32)        (a4w4_flatmm)

each with a shape-only ("fake") implementation, so that graph capture and shape propagation work
without running the kernels.  The real implementations call the library on the current stream and
raise if it is missing; there is no eager fallback.
"""
from . import api

_registered = False


def register():
    global _registered
    if _registered:
        return
    import torch

    def _cdt(out_fp32):
        return api.FP32 if out_fp32 else api.BF16

    def _odt(out_fp32):
        return torch.float32 if out_fp32 else torch.bfloat16

    @torch.library.custom_op("mi355_a8w8::gemm", mutates_args=())
    def gemm(a: torch.Tensor, b: torch.Tensor, sfa: torch.Tensor, sfb: torch.Tensor, scale_mode: int,
             out_fp32: bool) -> torch.Tensor:
        return api.gemm(a, b, sfa, sfb, scale_mode, c_dtype=_cdt(out_fp32))

    @gemm.register_fake
    def _(a, b, sfa, sfb, scale_mode, out_fp32):
        return a.new_empty((*a.shape[:-1], b.shape[-2]), dtype=_odt(out_fp32))

    @torch.library.custom_op("mi355_a8w8::flatmm", mutates_args=())
    def flatmm(a: torch.Tensor, b_shuffled: torch.Tensor, sfa: torch.Tensor, sfb: torch.Tensor, n: int, scale_mode: int,
               out_fp32: bool) -> torch.Tensor:
        return api.flatmm(a, b_shuffled, sfa, sfb, n, scale_mode=scale_mode, c_dtype=_cdt(out_fp32))

    @flatmm.register_fake
    def _(a, b_shuffled, sfa, sfb, n, scale_mode, out_fp32):
        return a.new_empty((*a.shape[:-1], n), dtype=_odt(out_fp32))

    @torch.library.custom_op("mi355_a8w8::gemm_a16w16", mutates_args=())
    def gemm_a16w16(a: torch.Tensor, b: torch.Tensor, out_fp32: bool) -> torch.Tensor:
        return api.gemm_a16w16(a, b, c_dtype=_cdt(out_fp32))

    @gemm_a16w16.register_fake
    def _(a, b, out_fp32):
        return a.new_empty((*a.shape[:-1], b.shape[-2]), dtype=_odt(out_fp32))

    @torch.library.custom_op("mi355_a8w8::quantize", mutates_args=())
    def quantize(x: torch.Tensor, scale_mode: int, group_rows: int) -> tuple[torch.Tensor, torch.Tensor]:
        return api.quantize(x, scale_mode, group_rows)

    @quantize.register_fake
    def _(x, scale_mode, group_rows):
        rows, k = x.shape
        q = x.new_empty((rows, k), dtype=torch.uint8)
        if scale_mode == api.TENSOR:
            s = x.new_empty((1,), dtype=torch.float32)
        elif scale_mode == api.ROWCOL:
            s = x.new_empty((rows,), dtype=torch.float32)
        elif scale_mode == api.BLOCK:
            s = x.new_empty((k // 128, rows) if group_rows == 1 else (rows // 128, k // 128), dtype=torch.float32)
        elif scale_mode == api.MX:
            s = x.new_empty((rows, k // 32), dtype=torch.uint8)
        else:
            s = x.new_empty((api.mx_tiled_bytes(rows, k),), dtype=torch.uint8)
        return q, s

    @torch.library.custom_op("mi355_a8w8::quantize_mxfp4", mutates_args=())
    def quantize_mxfp4(x: torch.Tensor, tiled: bool) -> tuple[torch.Tensor, torch.Tensor]:
        return api.quantize_mxfp4(x, tiled=tiled)

    @quantize_mxfp4.register_fake
    def _(x, tiled):
        rows, k = x.shape
        q = x.new_empty((rows, k // 2), dtype=torch.uint8)
        s = x.new_empty((api.mx_tiled_bytes(rows, k),) if tiled else (rows, k // 32), dtype=torch.uint8)
        return q, s

    @torch.library.custom_op("mi355_a8w8::gemm_a4w4", mutates_args=())
    def gemm_a4w4(a: torch.Tensor, b: torch.Tensor, sfa: torch.Tensor, sfb: torch.Tensor, scale_mode: int,
                  out_fp32: bool) -> torch.Tensor:
        return api.gemm_a4w4(a, b, sfa, sfb, scale_mode, c_dtype=_cdt(out_fp32))

    @gemm_a4w4.register_fake
    def _(a, b, sfa, sfb, scale_mode, out_fp32):
        return a.new_empty((a.shape[-2], b.shape[-2]), dtype=_odt(out_fp32))

    @torch.library.custom_op("mi355_a8w8::flatmm_a4w4", mutates_args=())
    def flatmm_a4w4(a: torch.Tensor, b_shuffled: torch.Tensor, sfa: torch.Tensor, sfb: torch.Tensor, n: int,
                    out_fp32: bool) -> torch.Tensor:
        return api.flatmm_a4w4(a, b_shuffled, sfa, sfb, n, c_dtype=_cdt(out_fp32))

    @flatmm_a4w4.register_fake
    def _(a, b_shuffled, sfa, sfb, n, out_fp32):
        return a.new_empty((a.shape[-2], n), dtype=_odt(out_fp32))

    _registered = True
