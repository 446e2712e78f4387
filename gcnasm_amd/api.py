"""ctypes front end of the C ABI declared in include/mi355_a8w8.h.

Argument names and meanings follow struct opus_gemm_kargs of the reference
(opus_gemm/block_scale_gemm/gemm_a8w8_blockscale_common.h:4-25): element strides, A [M,K]
and B [N,K] row-major E4M3 bytes, C [M,N].  Tensors are torch tensors used purely as
device-memory handles (data_ptr) plus the current HIP stream.
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
# MI355_A8W8_LIBRARY: another build of the same sources (a measurement build made with `make EXTRA=-D... OUT=...`),
# for A/B timings of one program against two libraries; unset, the library next to this file
_SO = os.environ.get("MI355_A8W8_LIBRARY") or os.path.join(_HERE, "libmi355a8w8.so")

TENSOR, ROWCOL, BLOCK, MX, MX_TILED = 0, 1, 2, 3, 4
BF16, FP32 = 0, 1
OCP, FNUZ = 0, 1


class A8W8Error(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        super().__init__(f"{where}: {status_string(status)} (status {status})")


class WeightHeader(ctypes.Structure):
    _fields_ = [("magic", ctypes.c_char * 8), ("version", ctypes.c_uint32), ("n", ctypes.c_uint32), ("k", ctypes.c_uint32),
                ("b_preshuffled", ctypes.c_uint32), ("scale_mode", ctypes.c_uint32), ("reserved", ctypes.c_uint32),
                ("b_bytes", ctypes.c_uint64), ("scale_bytes", ctypes.c_uint64), ("checksum", ctypes.c_uint64),
                ("reserved2", ctypes.c_uint64)]


class GemmArgs(ctypes.Structure):
    _fields_ = [
        ("a", ctypes.c_void_p), ("b", ctypes.c_void_p), ("c", ctypes.c_void_p),
        ("m", ctypes.c_int), ("n", ctypes.c_int), ("k", ctypes.c_int), ("batch", ctypes.c_int),
        ("stride_a", ctypes.c_int), ("stride_b", ctypes.c_int), ("stride_c", ctypes.c_int),
        ("stride_a_batch", ctypes.c_int), ("stride_b_batch", ctypes.c_int), ("stride_c_batch", ctypes.c_int),
        ("sfa", ctypes.c_void_p), ("sfb", ctypes.c_void_p),
        ("stride_sfa", ctypes.c_int), ("stride_sfb", ctypes.c_int),
        ("stride_sfa_batch", ctypes.c_int), ("stride_sfb_batch", ctypes.c_int),
        ("scale_mode", ctypes.c_int), ("c_dtype", ctypes.c_int), ("b_preshuffled", ctypes.c_int),
    ]


def library_path():
    return _SO


def build_library(verbose=False):
    """Compile the HIP sources for gfx950 with hipcc (cross-compiles without a GPU)."""
    subprocess.check_call(["make", "-C", os.path.join(_HERE, "csrc"), "-B"],
                          stdout=None if verbose else subprocess.DEVNULL,
                          stderr=None if verbose else subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    """The loaded C ABI.  Raises if the library has not been built; never substitutes a CPU path."""
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            raise FileNotFoundError(
                f"{_SO} is missing: build it with gcnasm_amd.build_library() or `make -C gcnasm_amd/csrc`")
        L = ctypes.CDLL(_SO)
        vp = ctypes.c_void_p
        L.a8w8_gemm.argtypes = [ctypes.POINTER(GemmArgs), vp]
        L.a8w8_gemm_blockscale.argtypes = [ctypes.POINTER(GemmArgs), vp]
        L.a16w16_gemm.argtypes = [ctypes.POINTER(GemmArgs), vp]
        L.a16w16_flatmm.argtypes = [ctypes.POINTER(GemmArgs), vp]
        L.a4w4_gemm.argtypes = [ctypes.POINTER(GemmArgs), vp]
        L.a4w4_flatmm.argtypes = [ctypes.POINTER(GemmArgs), vp]
        L.a4w4_quantize_mx.argtypes = [vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp, ctypes.c_int, vp]
        L.a8w8_flatmm.argtypes = [ctypes.POINTER(GemmArgs), vp]
        L.a8w8_preshuffle_b.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int]
        L.a8w8_unshuffle_b.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int]
        L.a8w8_preshuffle_b_device.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int, vp]
        L.a8w8_cvt_f32_to_e4m3.argtypes = [vp, vp, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, vp]
        L.a8w8_cvt_e4m3_to_f32.argtypes = [vp, vp, ctypes.c_size_t, ctypes.c_int, vp]
        L.a8w8_quantize.argtypes = [vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp, ctypes.c_int,
                                    ctypes.c_int, vp]
        L.a8w8_mx_tile_scales.argtypes = [vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp]
        L.a8w8_mx_tile_scales_ab.argtypes = [vp, ctypes.c_int, ctypes.c_int, vp, vp, ctypes.c_int, ctypes.c_int, vp,
                                             ctypes.c_int, vp]
        L.a8w8_mx_tiled_bytes.restype = ctypes.c_size_t
        L.a8w8_mx_tiled_bytes.argtypes = [ctypes.c_int, ctypes.c_int]
        L.a8w8_weight_scale_bytes.restype = ctypes.c_size_t
        L.a8w8_weight_scale_bytes.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.a8w8_weights_save.argtypes = [ctypes.c_char_p, vp, vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.a8w8_weights_info.argtypes = [ctypes.c_char_p, ctypes.POINTER(WeightHeader)]
        L.a8w8_weights_load.argtypes = [ctypes.c_char_p, vp, ctypes.c_size_t, vp, ctypes.c_size_t]
        L.a8w8_status_string.restype = ctypes.c_char_p
        L.a8w8_status_string.argtypes = [ctypes.c_int]
        L.a8w8_kernel_name.restype = ctypes.c_char_p
        L.a8w8_kernel_name.argtypes = [ctypes.POINTER(GemmArgs)]
        L.a8w8_version.restype = ctypes.c_int
        L.a8w8_init.argtypes = [ctypes.c_int]
        L.a8w8_hbm_read_probe.argtypes = [vp, ctypes.c_size_t, vp, vp]
        L.a8w8_route_override.argtypes = [ctypes.c_int]
        _lib = L
    return _lib


def status_string(status):
    return lib().a8w8_status_string(int(status)).decode()


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(status, where):
    if status != 0:
        raise A8W8Error(status, where)


def raw_gemm_args(a, b, c, sfa, sfb, m, n, k, scale_mode, c_dtype=BF16, batch=1, stride_a=None, stride_b=None,
                  stride_c=None, stride_sfa=None, stride_sfb=None, b_preshuffled=0, batch_strides=None):
    """Fill the C argument block from raw integers (device addresses)."""
    g = GemmArgs()
    g.a, g.b, g.c, g.sfa, g.sfb = a, b, c, sfa, sfb
    g.m, g.n, g.k, g.batch = m, n, k, batch
    g.stride_a = k if stride_a is None else stride_a
    g.stride_b = k if stride_b is None else stride_b
    g.stride_c = n if stride_c is None else stride_c
    if stride_sfa is None:
        stride_sfa = {TENSOR: 0, ROWCOL: 0, BLOCK: m, MX: k // 32}[scale_mode] if 0 <= scale_mode <= 3 else 0
    if stride_sfb is None:
        stride_sfb = {TENSOR: 0, ROWCOL: 1, BLOCK: k // 128, MX: k // 32}[scale_mode] if 0 <= scale_mode <= 3 else 0
    g.stride_sfa, g.stride_sfb = stride_sfa, stride_sfb
    if batch_strides is None:
        sfa_b = {TENSOR: 1, ROWCOL: m, BLOCK: m * (k // 128), MX: m * (k // 32),
                 MX_TILED: mx_tiled_bytes(m, k)}.get(scale_mode, 0)
        sfb_b = {TENSOR: 1, ROWCOL: n, BLOCK: (n // 128) * (k // 128), MX: n * (k // 32),
                 MX_TILED: mx_tiled_bytes(n, k)}.get(scale_mode, 0)
        batch_strides = (m * g.stride_a, n * g.stride_b, m * g.stride_c, sfa_b, sfb_b)
    (g.stride_a_batch, g.stride_b_batch, g.stride_c_batch, g.stride_sfa_batch, g.stride_sfb_batch) = batch_strides
    g.scale_mode, g.c_dtype, g.b_preshuffled = scale_mode, c_dtype, b_preshuffled
    return g


def mx_tiled_bytes(rows, k):
    """Size of one matrix's E8M0 scales in the MX_TILED layout."""
    return ((k + 511) // 512) * ((rows + 63) // 64) * 1024


def _out(c, shape, c_dtype, device):
    """The output tensor and its C type code: a caller's tensor decides the type (bf16 or fp32 only)."""
    import torch
    if c is None:
        return torch.empty(shape, dtype=torch.bfloat16 if c_dtype == BF16 else torch.float32, device=device), c_dtype
    if c.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"output tensor must be bfloat16 or float32, got {c.dtype}")
    if tuple(c.shape) != tuple(shape):
        raise ValueError(f"output tensor has shape {tuple(c.shape)}, expected {tuple(shape)}")
    return c, (BF16 if c.dtype == torch.bfloat16 else FP32)


def _check_operand(t, name, dims):
    """Operands are strided views of device memory whose rows are contiguous; anything else would be misread."""
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU")
    if t.dim() not in dims:
        raise ValueError(f"{name} must have {' or '.join(str(d) for d in dims)} dimensions, got {t.dim()}")
    if t.dim() >= 1 and t.shape[-1] > 1 and t.stride(-1) != 1:
        raise ValueError(f"{name}: the last dimension must be contiguous (stride {t.stride(-1)})")


def _check_scales(t, name, scale_mode):
    """Scale arrays are read with the strides their shape implies: they have to be contiguous, on the GPU, and of
    the element type of the scale mode (fp32, or uint8 for the E8M0 modes)."""
    import torch
    want = torch.uint8 if scale_mode in (MX, MX_TILED) else torch.float32
    if not t.is_cuda or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous GPU tensor")
    if t.dtype != want:
        raise TypeError(f"{name} must be {want} for this scale mode, got {t.dtype}")


def scale_elements(scale_mode, rows, k, weight_side):
    """Elements one batch entry's scale array holds for a matrix of `rows` rows (A: weight_side False, B: True), as the
    kernels index it with the default strides of raw_gemm_args."""
    if scale_mode == TENSOR:
        return 1
    if scale_mode == ROWCOL:
        return rows
    if scale_mode == BLOCK:
        return ((rows + 127) // 128 if weight_side else rows) * (k // 128)
    if scale_mode == MX:
        return rows * (k // 32)
    return mx_tiled_bytes(rows, k)


def _check_scale_sizes(sfa, sfb, scale_mode, m, n, k, batch, b_shared):
    """An undersized scale array would be read past its end on the device; weights shared by all batch entries come with
    one set of weight scales (a per-entry set would silently be used for entry 0 only)."""
    need_a = batch * scale_elements(scale_mode, m, k, False)
    per_b = scale_elements(scale_mode, n, k, True)
    need_b = per_b if b_shared else batch * per_b
    if sfa.numel() < need_a:
        raise ValueError(f"sfa holds {sfa.numel()} elements, this problem reads {need_a}")
    if sfb.numel() < need_b:
        raise ValueError(f"sfb holds {sfb.numel()} elements, this problem reads {need_b}")
    if b_shared and sfb.numel() >= batch * per_b and sfb.numel() > per_b:
        raise ValueError(f"b is shared by all {batch} batch entries but sfb holds a set of scales per entry; pass one set")


def _args_from_tensors(a, b, sfa, sfb, scale_mode, c, c_dtype, b_preshuffled, n=None, scaled=True):
    _check_operand(a, "a", (2, 3))
    _check_operand(b, "b", (1, 2) if b_preshuffled else (2, 3))
    if scaled:
        _check_scales(sfa, "sfa", scale_mode)
        _check_scales(sfb, "sfb", scale_mode)
    batch = a.shape[0] if a.dim() == 3 else 1
    m, k = a.shape[-2], a.shape[-1]
    if n is None:
        n = b.shape[-2]
    shape = (batch, m, n) if a.dim() == 3 else (m, n)
    c, c_dtype = _out(c, shape, c_dtype, a.device)
    if c.dim() >= 2 and c.shape[-1] > 1 and c.stride(-1) != 1:
        raise ValueError("c: the last dimension must be contiguous")
    g = raw_gemm_args(a.data_ptr(), b.data_ptr(), c.data_ptr(), sfa.data_ptr(), sfb.data_ptr(), m, n, k, scale_mode,
                      c_dtype, batch, stride_a=a.stride(-2), stride_b=(k if b_preshuffled else b.stride(-2)),
                      stride_c=c.stride(-2), b_preshuffled=b_preshuffled)
    if a.dim() == 3:
        g.stride_a_batch, g.stride_c_batch = a.stride(0), c.stride(0)
        if b_preshuffled:
            # flat shuffled weights: of every batch entry back to back, or one matrix shared by all of them
            per_entry = n * k * a.element_size() // b.element_size()
            if b.numel() == batch * per_entry:
                g.stride_b_batch = n * k
            elif b.numel() == per_entry:
                g.stride_b_batch = 0
                g.stride_sfb_batch = 0
            else:
                raise ValueError(f"shuffled b holds {b.numel()} elements, expected {per_entry} or {batch} x {per_entry}")
        elif b.dim() == 3:
            if b.shape[0] != batch:
                raise ValueError(f"b has {b.shape[0]} batch entries, a has {batch}")
            g.stride_b_batch = b.stride(0)
        else:
            # one weight matrix shared by every batch entry, and with it one set of weight scales
            g.stride_b_batch = 0
            g.stride_sfb_batch = 0
    if scaled:
        _check_scale_sizes(sfa, sfb, scale_mode, m, n, k, batch, b_shared=(batch > 1 and g.stride_b_batch == 0))
    return g, c


def gemm(a, b, sfa, sfb, scale_mode, c=None, c_dtype=BF16, n=None):
    """C = dequant(A) @ dequant(B)^T through a8w8_gemm.  a [.., M, K] u8, b [.., N, K] u8 on the GPU; with `n` given,
    b is the flat pre-shuffled weight (preshuffle_b_device) of n rows."""
    g, c = _args_from_tensors(a, b, sfa, sfb, scale_mode, c, c_dtype, 0 if n is None else 1, n=n)
    _check(lib().a8w8_gemm(ctypes.byref(g), _stream()), "a8w8_gemm")
    return c


def gemm_a16w16(a, b, c=None, c_dtype=BF16, n=None):
    """C = A @ B^T for bf16 a [.., M, K] and b [.., N, K] (torch.bfloat16 on the GPU) through a16w16_gemm; with `n`
    given, b is the flat pre-shuffled weight of n rows (preshuffle_b_bf16_device)."""
    g, c = _args_from_tensors(a, b, a, b, TENSOR, c, c_dtype, 0 if n is None else 1, n=n, scaled=False)
    _check(lib().a16w16_gemm(ctypes.byref(g), _stream()), "a16w16_gemm")
    return c


def preshuffle_b_bf16_device(b):
    """bf16 weights [N, K] on the GPU -> the pre-shuffled byte layout a16w16_flatmm streams (flat uint8 tensor)."""
    import torch
    n, k = b.shape
    return preshuffle_b_device(b.contiguous().view(torch.uint8).view(n, 2 * k))


def flatmm_a16w16(a, b_shuffled, n, c=None, c_dtype=BF16):
    """Skinny-M bf16 GEMM over weights from preshuffle_b_bf16_device."""
    g, c = _args_from_tensors(a, b_shuffled, a, a, TENSOR, c, c_dtype, 1, n=n, scaled=False)
    _check(lib().a16w16_flatmm(ctypes.byref(g), _stream()), "a16w16_flatmm")
    return c


def quantize_mxfp4(x, tiled=False):
    """fp32 [rows, K] -> (packed E2M1 bytes [rows, K/2], E8M0 scales row-major [rows, K/32] or tiled)."""
    import torch
    rows, k = x.shape
    q = torch.empty((rows, k // 2), dtype=torch.uint8, device=x.device)
    s = torch.empty(mx_tiled_bytes(rows, k) if tiled else (rows, k // 32), dtype=torch.uint8, device=x.device)
    _check(lib().a4w4_quantize_mx(x.data_ptr(), rows, k, x.stride(0), q.data_ptr(), s.data_ptr(), int(tiled), _stream()),
           "a4w4_quantize_mx")
    return q, s


def gemm_a4w4(a, b, sfa, sfb, scale_mode=MX_TILED, c=None, c_dtype=BF16, n=None):
    """MXFP4 GEMM through a4w4_gemm: a [M, K/2], b [N, K/2] packed E2M1 (uint8 on the GPU); with `n` given, b is the
    flat pre-shuffled weight of n rows (preshuffle_b_device on the packed bytes)."""
    m, k = a.shape[-2], a.shape[-1] * 2
    shuffled = n is not None
    if not shuffled:
        n = b.shape[-2]
    c, c_dtype = _out(c, (m, n), c_dtype, a.device)
    g = raw_gemm_args(a.data_ptr(), b.data_ptr(), c.data_ptr(), sfa.data_ptr(), sfb.data_ptr(), m, n, k, scale_mode, c_dtype,
                      stride_a=a.stride(-2) * 2, stride_b=(k if shuffled else b.stride(-2) * 2), stride_c=c.stride(-2),
                      b_preshuffled=int(shuffled))
    _check(lib().a4w4_gemm(ctypes.byref(g), _stream()), "a4w4_gemm")
    return c


def flatmm_a4w4(a, b_shuffled, sfa_tiled, sfb_tiled, n, c=None, c_dtype=BF16):
    """MXFP4 skinny-M GEMM through a4w4_flatmm: a [M, K/2] packed E2M1 with M <= 128, b_shuffled from
    preshuffle_b_device on the packed weight bytes [N, K/2], both scale arrays in the MX_TILED layout."""
    m, k = a.shape[-2], a.shape[-1] * 2
    c, c_dtype = _out(c, (m, n), c_dtype, a.device)
    g = raw_gemm_args(a.data_ptr(), b_shuffled.data_ptr(), c.data_ptr(), sfa_tiled.data_ptr(), sfb_tiled.data_ptr(), m, n, k,
                      MX_TILED, c_dtype, stride_a=a.stride(-2) * 2, stride_b=k, stride_c=c.stride(-2), b_preshuffled=1)
    _check(lib().a4w4_flatmm(ctypes.byref(g), _stream()), "a4w4_flatmm")
    return c


def gemm_blockscale(a, b, sfa, sfb, c=None, c_dtype=FP32):
    """The reference's block-scale GEMM (1x128 / 128x128 scales), fp32 C by default as there."""
    g, c = _args_from_tensors(a, b, sfa, sfb, BLOCK, c, c_dtype, 0)
    _check(lib().a8w8_gemm_blockscale(ctypes.byref(g), _stream()), "a8w8_gemm_blockscale")
    return c


def flatmm(a, b_shuffled, sfa, sfb, n, scale_mode=ROWCOL, c=None, c_dtype=BF16):
    """Skinny-M GEMM over weights in the a8w8_preshuffle_b layout (flat u8 tensor of n*k bytes); scale_mode ROWCOL,
    TENSOR or MX_TILED (MXFP8: both scale arrays in the tiled layout)."""
    g, c = _args_from_tensors(a, b_shuffled, sfa, sfb, scale_mode, c, c_dtype, 1, n=n)
    _check(lib().a8w8_flatmm(ctypes.byref(g), _stream()), "a8w8_flatmm")
    return c


def preshuffle_b(b_np):
    """Host pre-shuffle of a numpy [N, K] uint8 weight; returns a flat uint8 array."""
    import numpy as np
    b_np = np.ascontiguousarray(b_np, dtype=np.uint8)
    n, k = b_np.shape
    out = np.empty(n * k, np.uint8)
    _check(lib().a8w8_preshuffle_b(b_np.ctypes.data, out.ctypes.data, n, k), "a8w8_preshuffle_b")
    return out


def unshuffle_b(bs_np, n, k):
    import numpy as np
    bs_np = np.ascontiguousarray(bs_np, dtype=np.uint8)
    out = np.empty((n, k), np.uint8)
    _check(lib().a8w8_unshuffle_b(bs_np.ctypes.data, out.ctypes.data, n, k), "a8w8_unshuffle_b")
    return out


def preshuffle_b_device(b):
    import torch
    n, k = b.shape
    out = torch.empty(n * k, dtype=torch.uint8, device=b.device)
    _check(lib().a8w8_preshuffle_b_device(b.data_ptr(), out.data_ptr(), n, k, _stream()), "a8w8_preshuffle_b_device")
    return out


def cvt_f32_to_e4m3(x, dialect=OCP, clamp240=False):
    import torch
    x = x.contiguous()
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    _check(lib().a8w8_cvt_f32_to_e4m3(x.data_ptr(), out.data_ptr(), x.numel(), dialect, int(clamp240), _stream()),
           "a8w8_cvt_f32_to_e4m3")
    return out


def cvt_e4m3_to_f32(codes, dialect=OCP):
    import torch
    codes = codes.contiguous()
    out = torch.empty(codes.shape, dtype=torch.float32, device=codes.device)
    _check(lib().a8w8_cvt_e4m3_to_f32(codes.data_ptr(), out.data_ptr(), codes.numel(), dialect, _stream()),
           "a8w8_cvt_e4m3_to_f32")
    return out


def quantize(x, scale_mode, group_rows=1):
    """fp32 [rows, K] -> (E4M3 bytes [rows, K], scales in the layout a8w8_gemm reads)."""
    import torch
    rows, k = x.shape
    q = torch.empty((rows, k), dtype=torch.uint8, device=x.device)
    if scale_mode == TENSOR:
        s = torch.empty(1, dtype=torch.float32, device=x.device)
    elif scale_mode == ROWCOL:
        s = torch.empty(rows, dtype=torch.float32, device=x.device)
    elif scale_mode == BLOCK and group_rows == 1:
        s = torch.empty((k // 128, rows), dtype=torch.float32, device=x.device)
    elif scale_mode == BLOCK:
        s = torch.empty((rows // 128, k // 128), dtype=torch.float32, device=x.device)
    elif scale_mode == MX:
        s = torch.empty((rows, k // 32), dtype=torch.uint8, device=x.device)
    elif scale_mode == MX_TILED:
        s = torch.empty(mx_tiled_bytes(rows, k), dtype=torch.uint8, device=x.device)
    else:
        raise A8W8Error(-6, "a8w8_quantize")
    _check(lib().a8w8_quantize(x.data_ptr(), rows, k, x.stride(0), q.data_ptr(), s.data_ptr(), scale_mode, group_rows,
                               _stream()), "a8w8_quantize")
    return q, s


def mx_tile_scales(sf, out=None):
    """Row-major E8M0 scales [rows, K/32] (u8, on the GPU) -> the MX_TILED layout (flat u8 tensor)."""
    import torch
    rows, kb = sf.shape
    if out is None:
        out = torch.empty(mx_tiled_bytes(rows, kb * 32), dtype=torch.uint8, device=sf.device)
    _check(lib().a8w8_mx_tile_scales(sf.data_ptr(), rows, kb * 32, sf.stride(0), out.data_ptr(), _stream()),
           "a8w8_mx_tile_scales")
    return out


def mx_tile_scales_ab(sfa, sfb):
    """Both scale arrays of a GEMM ([M, K/32] and [N, K/32] u8) -> MX_TILED, one launch."""
    import torch
    m, kb = sfa.shape
    n = sfb.shape[0]
    ta = torch.empty(mx_tiled_bytes(m, kb * 32), dtype=torch.uint8, device=sfa.device)
    tb = torch.empty(mx_tiled_bytes(n, kb * 32), dtype=torch.uint8, device=sfb.device)
    _check(lib().a8w8_mx_tile_scales_ab(sfa.data_ptr(), m, sfa.stride(0), ta.data_ptr(), sfb.data_ptr(), n,
                                        sfb.stride(0), tb.data_ptr(), kb * 32, _stream()), "a8w8_mx_tile_scales_ab")
    return ta, tb


def save_weights(path, b_np, scale_np, n, k, scale_mode, b_preshuffled=False):
    """Write quantised weights (numpy uint8, row-major [n, k] or pre-shuffled flat) and their scales to a file."""
    import numpy as np
    b_np = np.ascontiguousarray(b_np, dtype=np.uint8)
    scale_np = np.ascontiguousarray(scale_np)
    assert b_np.size == n * k and scale_np.nbytes == lib().a8w8_weight_scale_bytes(n, k, scale_mode)
    _check(lib().a8w8_weights_save(os.fsencode(path), b_np.ctypes.data, scale_np.ctypes.data, n, k, int(b_preshuffled),
                                   scale_mode), "a8w8_weights_save")


def load_weights(path):
    """-> (header, weights uint8 array, scales array: float32, or uint8 for the MX modes)."""
    import numpy as np
    h = WeightHeader()
    _check(lib().a8w8_weights_info(os.fsencode(path), ctypes.byref(h)), "a8w8_weights_info")
    b = np.empty(h.b_bytes, np.uint8)
    raw = np.empty(h.scale_bytes, np.uint8)
    _check(lib().a8w8_weights_load(os.fsencode(path), b.ctypes.data, b.nbytes, raw.ctypes.data, raw.nbytes), "a8w8_weights_load")
    scales = raw if h.scale_mode in (MX, MX_TILED) else raw.view(np.float32)
    return h, (b if h.b_preshuffled else b.reshape(h.n, h.k)), scales


def init(device=-1):
    """Explicit one-time set-up of a device (the current one by default); see a8w8_init."""
    _check(lib().a8w8_init(int(device)), "a8w8_init")


def kernel_name(g):
    r = lib().a8w8_kernel_name(ctypes.byref(g))
    return r.decode() if r else None
