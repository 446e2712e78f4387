"""CPU oracle for the A8W8 FP8 GEMM path -- TEST INFRASTRUCTURE ONLY.

numpy/ctypes front end of ``a8w8_oracle.c`` (a plain-C restatement of the reference's
host arithmetic).  Only the test suite, the smoke check and the benchmark's CPU-baseline
leg may import this package; the product library never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liba8w8_oracle.so")

_u8p = ctypes.POINTER(ctypes.c_uint8)
_f32p = ctypes.POINTER(ctypes.c_float)
_i32p = ctypes.POINTER(ctypes.c_int)
_u16p = ctypes.POINTER(ctypes.c_uint16)


def build(force=False):
    """Compile the C restatement with gcc (seconds)."""
    src = os.path.join(_HERE, "a8w8_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liba8w8_oracle.so"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        L.orc_e4m3_fnuz_decode.restype = ctypes.c_float
        L.orc_e4m3_fnuz_decode.argtypes = [ctypes.c_uint8]
        L.orc_e4m3_ocp_decode.restype = ctypes.c_float
        L.orc_e4m3_ocp_decode.argtypes = [ctypes.c_uint8]
        L.orc_e8m0_decode.restype = ctypes.c_float
        L.orc_e8m0_decode.argtypes = [ctypes.c_uint8]
        L.orc_f8_cast_from_f8_bits.restype = ctypes.c_uint32
        L.orc_f8_cast_from_f8_bits.argtypes = [ctypes.c_uint8, ctypes.c_int]
        L.orc_e4m3_ocp_encode.restype = ctypes.c_uint8
        L.orc_e4m3_ocp_encode.argtypes = [ctypes.c_float]
        L.orc_e4m3_fnuz_encode.restype = ctypes.c_uint8
        L.orc_e4m3_fnuz_encode.argtypes = [ctypes.c_float]
        L.orc_cvt_fp8_clamp240.restype = ctypes.c_uint8
        L.orc_cvt_fp8_clamp240.argtypes = [ctypes.c_float, ctypes.c_int]
        L.orc_pk_cvt_fp8x4.restype = ctypes.c_uint32
        L.orc_pk_cvt_fp8x4.argtypes = [_f32p, ctypes.c_int]
        L.orc_f32_to_bf16.restype = ctypes.c_uint16
        L.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        L.orc_decode_vec.argtypes = [_u8p, _f32p, ctypes.c_size_t, ctypes.c_int]
        L.orc_encode_vec.argtypes = [_f32p, _u8p, ctypes.c_size_t, ctypes.c_int, ctypes.c_int]
        L.orc_convert_vec.argtypes = [_f32p, _u8p, ctypes.c_size_t, ctypes.c_int]
        L.orc_e4m3_ocp_encode_hw.restype = ctypes.c_uint8
        L.orc_e4m3_ocp_encode_hw.argtypes = [ctypes.c_float]
        L.orc_bf16_vec.argtypes = [_f32p, _u16p, ctypes.c_size_t]
        L.orc_gemm_ref.argtypes = [_u8p, _u8p, _f32p, _f32p, _f32p] + [ctypes.c_int] * 14
        L.orc_gemm_ref_mx.argtypes = [_u8p, _u8p, _u8p, _u8p, _f32p] + [ctypes.c_int] * 11
        L.orc_gemm_probe.argtypes = ([_u8p, _u8p, ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 9
                                     + [_i32p, _i32p, ctypes.c_int, _f32p])
        L.orc_preshuffle_index.restype = ctypes.c_size_t
        L.orc_preshuffle_index.argtypes = [ctypes.c_int] * 3
        L.orc_preshuffle_b.argtypes = [_u8p, _u8p, ctypes.c_int, ctypes.c_int]
        L.orc_unshuffle_b.argtypes = [_u8p, _u8p, ctypes.c_int, ctypes.c_int]
        L.orc_mx_tiled_bytes.restype = ctypes.c_size_t
        L.orc_mx_tiled_bytes.argtypes = [ctypes.c_int, ctypes.c_int]
        L.orc_mx_tile_scales.argtypes = [_u8p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _u8p]
        L.orc_mx_untile_scales.argtypes = [_u8p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _u8p]
        L.orc_e2m1_decode.restype = ctypes.c_float
        L.orc_e2m1_decode.argtypes = [ctypes.c_uint8]
        L.orc_e2m1_encode.restype = ctypes.c_uint8
        L.orc_e2m1_encode.argtypes = [ctypes.c_float]
        L.orc_gemm_ref_mxfp4.argtypes = [_u8p, _u8p, _u8p, _u8p, _f32p] + [ctypes.c_int] * 5
        L.orc_quant_mxfp4.argtypes = [_f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _u8p, _u8p]
        L.orc_gemm_bf16_ref.argtypes = [_u16p, _u16p, _f32p] + [ctypes.c_int] * 6
        L.orc_quant_tensor.argtypes = [_f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _u8p, _f32p]
        L.orc_quant_rowwise.argtypes = [_f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _u8p, _f32p]
        L.orc_quant_block.argtypes = [_f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _u8p, _f32p, ctypes.c_int]
        L.orc_quant_mx.argtypes = [_f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _u8p, _u8p]
        L.orc_flatmm_ref.argtypes = [_u8p, _u8p, _f32p, _f32p, _f32p] + [ctypes.c_int] * 5
        L.orc_count_abs_mismatch.restype = ctypes.c_long
        L.orc_count_abs_mismatch.argtypes = [_f32p, _f32p, ctypes.c_size_t, ctypes.c_float]
        L.orc_num_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def _p(arr, ty):
    return arr.ctypes.data_as(ty)


def _c(arr, dtype):
    arr = np.ascontiguousarray(arr, dtype=dtype)
    return arr


OCP, FNUZ = 0, 1

# scale-mode numbers of the library ABI
TENSOR, ROWCOL, BLOCK, MX = 0, 1, 2, 3


def decode(codes, dialect=OCP):
    codes = _c(codes, np.uint8)
    out = np.empty(codes.shape, np.float32)
    lib().orc_decode_vec(_p(codes, _u8p), _p(out, _f32p), codes.size, dialect)
    return out


def encode(x, dialect=OCP, clamp240=False):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint8)
    lib().orc_encode_vec(_p(x, _f32p), _p(out, _u8p), x.size, dialect, int(clamp240))
    return out


def convert(x, dialect=OCP):
    """The device's unclamped convert: the gfx950 instruction (OCP, not saturating: overflow and Inf
    give the NaN code) or, for FNUZ, the saturating conversion of __hip_fp8_e4m3_fnuz."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint8)
    lib().orc_convert_vec(_p(x, _f32p), _p(out, _u8p), x.size, dialect)
    return out


def cast_from_f8_bits(code, negative_zero_nan):
    return lib().orc_f8_cast_from_f8_bits(int(code), int(negative_zero_nan))


def pk_cvt_fp8x4(s4, dialect=OCP):
    s4 = _c(s4, np.float32)
    assert s4.size == 4
    return lib().orc_pk_cvt_fp8x4(_p(s4, _f32p), dialect)


def e8m0_decode(b):
    return lib().orc_e8m0_decode(int(b))


def to_bf16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_bf16_vec(_p(x, _f32p), _p(out, _u16p), x.size)
    return out


def bf16_bits_to_f32(h):
    return (np.ascontiguousarray(h, np.uint16).astype(np.uint32) << 16).view(np.float32)


def round_bf16(x):
    """fp32 -> bf16 (RNE) -> fp32."""
    return bf16_bits_to_f32(to_bf16_bits(x))


def _grouping(mode, m, n, k):
    """gemm_ref (group_m, group_n, group_k, stride_sfa, stride_sfb) for a scale mode."""
    if mode == TENSOR:
        return m, n, k, 0, 0
    if mode == ROWCOL:
        return 1, 1, k, 0, 1
    if mode == BLOCK:
        return 1, 128, 128, m, k // 128
    raise ValueError(mode)


def gemm_ref(a, b, sfa, sfb, mode, rows=None, decode_per_mac=False):
    """C[rows] (fp32) of the reference CPU GEMM.  a [M,K] u8, b [N,K] u8."""
    a = _c(a, np.uint8)
    b = _c(b, np.uint8)
    m, k = a.shape
    n = b.shape[0]
    r0, r1 = rows if rows is not None else (0, m)
    c = np.zeros((m, n), np.float32)
    if mode == MX:
        sfa = _c(sfa, np.uint8)
        sfb = _c(sfb, np.uint8)
        lib().orc_gemm_ref_mx(_p(a, _u8p), _p(b, _u8p), _p(sfa, _u8p), _p(sfb, _u8p), _p(c, _f32p),
                              m, n, k, k, k, n, sfa.shape[-1], sfb.shape[-1], r0, r1, int(decode_per_mac))
    else:
        sfa = _c(sfa, np.float32)
        sfb = _c(sfb, np.float32)
        gm, gn, gk, ssa, ssb = _grouping(mode, m, n, k)
        lib().orc_gemm_ref(_p(a, _u8p), _p(b, _u8p), _p(sfa, _f32p), _p(sfb, _f32p), _p(c, _f32p),
                           m, n, k, k, k, n, ssa, ssb, gm, gn, gk, r0, r1, int(decode_per_mac))
    return c[r0:r1]


def gemm_probe(a, b, sfa, sfb, mode, pi, pj):
    a = _c(a, np.uint8)
    b = _c(b, np.uint8)
    m, k = a.shape
    n = b.shape[0]
    pi = _c(pi, np.int32)
    pj = _c(pj, np.int32)
    out = np.empty(pi.size, np.float32)
    if mode == MX:
        sfa = _c(sfa, np.uint8)
        sfb = _c(sfb, np.uint8)
        gm = gn = 1
        gk = 32
        ssa, ssb = sfa.shape[-1], sfb.shape[-1]
    else:
        sfa = _c(sfa, np.float32)
        sfb = _c(sfb, np.float32)
        gm, gn, gk, ssa, ssb = _grouping(mode, m, n, k)
    lib().orc_gemm_probe(_p(a, _u8p), _p(b, _u8p), sfa.ctypes.data, sfb.ctypes.data, k, k, k, ssa, ssb,
                         gm, gn, gk, mode, _p(pi, _i32p), _p(pj, _i32p), pi.size, _p(out, _f32p))
    return out


def preshuffle_b(b):
    b = _c(b, np.uint8)
    n, k = b.shape
    out = np.empty(n * k, np.uint8)
    lib().orc_preshuffle_b(_p(b, _u8p), _p(out, _u8p), n, k)
    return out


def unshuffle_b(bs, n, k):
    bs = _c(bs, np.uint8)
    out = np.empty((n, k), np.uint8)
    lib().orc_unshuffle_b(_p(bs, _u8p), _p(out, _u8p), n, k)
    return out


def mx_tiled_bytes(rows, k):
    return lib().orc_mx_tiled_bytes(rows, k)


def mx_tile_scales(sf):
    """[rows, K/32] u8 -> flat u8 in the library's tiled MX scale layout."""
    sf = _c(sf, np.uint8)
    rows, kb = sf.shape
    out = np.empty(mx_tiled_bytes(rows, kb * 32), np.uint8)
    lib().orc_mx_tile_scales(_p(sf, _u8p), rows, kb * 32, kb, _p(out, _u8p))
    return out


def mx_untile_scales(tiled, rows, k):
    tiled = _c(tiled, np.uint8)
    out = np.zeros((rows, k // 32), np.uint8)
    lib().orc_mx_untile_scales(_p(tiled, _u8p), rows, k, k // 32, _p(out, _u8p))
    return out


def e2m1_decode_packed(q):
    """[rows, K/2] packed E2M1 bytes -> fp32 [rows, K] (even K in the low nibble)."""
    q = _c(q, np.uint8)
    table = np.array([lib().orc_e2m1_decode(c) for c in range(16)], np.float32)
    out = np.empty(q.shape[:-1] + (q.shape[-1] * 2,), np.float32)
    out[..., 0::2] = table[q & 15]
    out[..., 1::2] = table[q >> 4]
    return out


def gemm_ref_mxfp4(a, b, ea, eb, rows=None):
    a, b, ea, eb = _c(a, np.uint8), _c(b, np.uint8), _c(ea, np.uint8), _c(eb, np.uint8)
    m, n, k = a.shape[0], b.shape[0], a.shape[1] * 2
    r0, r1 = rows if rows is not None else (0, m)
    c = np.zeros((m, n), np.float32)
    lib().orc_gemm_ref_mxfp4(_p(a, _u8p), _p(b, _u8p), _p(ea, _u8p), _p(eb, _u8p), _p(c, _f32p), m, n, k, r0, r1)
    return c[r0:r1]


def quantize_mxfp4(x):
    x = _c(x, np.float32)
    rows, k = x.shape
    q = np.empty((rows, k // 2), np.uint8)
    s = np.empty((rows, k // 32), np.uint8)
    lib().orc_quant_mxfp4(_p(x, _f32p), rows, k, k, _p(q, _u8p), _p(s, _u8p))
    return q, s


def gemm_bf16_ref(a_bits, b_bits):
    """fp32 C of the bf16 GEMM; a_bits [M, K], b_bits [N, K] uint16 bf16 patterns."""
    a_bits = _c(a_bits, np.uint16)
    b_bits = _c(b_bits, np.uint16)
    m, k = a_bits.shape
    n = b_bits.shape[0]
    c = np.empty((m, n), np.float32)
    lib().orc_gemm_bf16_ref(_p(a_bits, _u16p), _p(b_bits, _u16p), _p(c, _f32p), m, n, k, k, k, n)
    return c


def quantize(x, mode, group_rows=1):
    """fp32 [rows, k] -> (E4M3 bytes, scales in the layout gemm_ref reads for `mode`)."""
    x = _c(x, np.float32)
    rows, k = x.shape
    q = np.empty((rows, k), np.uint8)
    if mode == TENSOR:
        s = np.empty(1, np.float32)
        lib().orc_quant_tensor(_p(x, _f32p), rows, k, k, _p(q, _u8p), _p(s, _f32p))
    elif mode == ROWCOL:
        s = np.empty(rows, np.float32)
        lib().orc_quant_rowwise(_p(x, _f32p), rows, k, k, _p(q, _u8p), _p(s, _f32p))
    elif mode == BLOCK:
        s = np.empty((k // 128, rows) if group_rows == 1 else (rows // 128, k // 128), np.float32)
        lib().orc_quant_block(_p(x, _f32p), rows, k, k, _p(q, _u8p), _p(s, _f32p), group_rows)
    elif mode == MX:
        s = np.empty((rows, k // 32), np.uint8)
        lib().orc_quant_mx(_p(x, _f32p), rows, k, k, _p(q, _u8p), _p(s, _u8p))
    else:
        raise ValueError(mode)
    return q, s


def flatmm_ref(a, bshuf, sfa, sfb, n):
    a = _c(a, np.uint8)
    bshuf = _c(bshuf, np.uint8)
    sfa = _c(sfa, np.float32)
    sfb = _c(sfb, np.float32)
    m, k = a.shape
    c = np.zeros((m, n), np.float32)
    lib().orc_flatmm_ref(_p(a, _u8p), _p(bshuf, _u8p), _p(sfa, _f32p), _p(sfb, _f32p), _p(c, _f32p),
                         m, n, k, k, n)
    return c


def count_abs_mismatch(ref, out, thr=1e-3):
    ref = _c(ref, np.float32)
    out = _c(out, np.float32)
    return lib().orc_count_abs_mismatch(_p(ref, _f32p), _p(out, _f32p), ref.size, thr)


def num_threads():
    return lib().orc_num_threads()
