/*
 * libmi355a8w8 -- A8W8 (FP8 E4M3 x FP8 E4M3) quantised GEMM for MI355X (gfx950), C ABI.
 *
 * Plain pointers and sizes only.  Every device pointer is memory the caller owns on the
 * current HIP device; the library allocates nothing and never frees caller memory.
 * Calls are asynchronous on the supplied hipStream_t (passed as void*, NULL = the default
 * stream, which is what the reference launches on); they do not synchronise.  Errors are
 * returned as negative a8w8_status values; nothing throws or exits across this boundary.
 *
 * The entry points stand in for the kernel-launch contract of carlushuang/gcnasm's FP8
 * GEMM demos.  Citations give the reference file:line (relative to its checkout) that
 * each one replaces.
 */
#ifndef MI355_A8W8_H
#define MI355_A8W8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define A8W8_API __attribute__((visibility("default")))

typedef enum {
    A8W8_OK = 0,
    A8W8_ERR_NULL_POINTER = -1,   /* a required pointer is NULL                            */
    A8W8_ERR_BAD_SHAPE = -2,      /* non-positive m/n/k/batch (host.cc:175-178)            */
    A8W8_ERR_BAD_GROUP = -3,      /* n or k not a multiple of the scale group (host.cc:183-187) */
    A8W8_ERR_BAD_STRIDE = -4,     /* a leading dimension smaller than the row it spans      */
    A8W8_ERR_MISALIGNED = -5,     /* pointer or stride not aligned as the kernel needs      */
    A8W8_ERR_BAD_MODE = -6,       /* unknown scale_mode / c_dtype / dialect, or a combination
                                     the entry point does not implement                    */
    A8W8_ERR_TOO_LARGE = -7,      /* an offset would not fit the 32-bit addressing in use   */
    A8W8_ERR_LAUNCH = -8,         /* the kernel launch itself returned an error             */
    A8W8_ERR_NO_DEVICE = -9,      /* no gfx950 device is current                            */
    A8W8_ERR_IO = -10,            /* a weight file could not be opened, read or written     */
    A8W8_ERR_BAD_FILE = -11       /* not a weight file of this version, truncated, or its
                                     checksum does not match                                */
} a8w8_status;

/* How the dequantisation scales are laid out.  All fp32 unless stated.
 *   TENSOR  sfa[1], sfb[1]
 *   ROWCOL  sfa[m] (per row of A, "per token"), sfb[n] (per row of B, "per channel")
 *   BLOCK   the reference layout (host.cc:78-79, 244-245):
 *             sfa[g*stride_sfa + i]          one scale per 1 x 128 block of A, g = k/128
 *             sfb[(j/128)*stride_sfb + g]    one scale per 128 x 128 block of B
 *   MX      uint8 E8M0 exponents, one per 32 K-elements, value 2^(e-127):
 *             sfa[i*stride_sfa + k/32], sfb[j*stride_sfb + k/32]
 *   MX_TILED  the same exponents re-arranged by a8w8_mx_tile_scales (or written that way by
 *             a8w8_quantize) so that the GEMM reads them as whole cache lines; stride_sfa /
 *             stride_sfb are ignored.  a8w8_mx_tiled_bytes(rows, k) =
 *             ceil(k/512) * ceil(rows/64) * 1024 bytes per array (rows = m or n), laid out as
 *                 [k/512][ceil(rows/64)][pair: 2][r16: 16][g: 4][jp: 2][par: 2][s: 2]   (one byte each)
 *             With kb = k/32 (the 32-wide K block) and rr = r % 64, the exponent of (row r, block kb) is byte
 *                 ((((kb/16) * ceil(rows/64) + r/64) * 2 + (kb/8)%2) * 64 + (4*((rr/8)%4) + rr%4) * 4 + kb%4) * 8
 *                   + (rr/32) * 4 + ((rr/4)%2) * 2 + (kb/4)%2
 *             (pair = (kb/8)%2, r16 = 4*((rr/8)%4) + rr%4, g = kb%4, jp = rr/32, par = (rr/4)%2, s = (kb/4)%2).
 *             Positions no (row, block) owns (rows past m or n, blocks past k) hold 127, the identity scale.
 *             With row-major scales every 16 bytes the kernel needs sit in a different 128-byte line. */
typedef enum {
    A8W8_SCALE_TENSOR = 0,
    A8W8_SCALE_ROWCOL = 1,
    A8W8_SCALE_BLOCK_1x128_128x128 = 2,
    A8W8_SCALE_MX_E8M0_1x32 = 3,
    A8W8_SCALE_MX_E8M0_TILED = 4
} a8w8_scale_mode;

typedef enum { A8W8_C_BF16 = 0, A8W8_C_FP32 = 1 } a8w8_c_dtype;
typedef enum { A8W8_E4M3_OCP = 0, A8W8_E4M3_FNUZ = 1 } a8w8_fp8_dialect;

/* Argument block.  A superset of struct opus_gemm_kargs
 * (opus_gemm/block_scale_gemm/gemm_a8w8_blockscale_common.h:4-25) with the same field
 * meanings: A is [batch, m, k] row-major, B is [batch, n, k] row-major (the column-major
 * K x N weight), C is [batch, m, n]; every stride counts ELEMENTS (common.h:12-17).
 * A and B hold OCP E4M3 bytes.  C[i,j] = sum_k A[i,k] * B[j,k] * scale.
 * Sizes (else A8W8_ERR_TOO_LARGE): one batch entry of A and of B spans less than 2 GiB, batch <= 65535, and, for
 * problems that run on the two 256 x 256-tile kernels (a8w8_kernel_name: gemm_a8w8_wide, gemm_a8w8_persist), whose
 * tiles are addressed with unsigned 32-bit byte offsets, (255 stride_c + 256) * sizeof(C element) < 2^32, i.e.
 * stride_c <= 4,210,751 for fp32 and <= 8,421,503 for bf16; the other kernels take any stride_c. */
typedef struct {
    const void* a;
    const void* b;
    void* c;
    int m, n, k, batch;
    int stride_a, stride_b, stride_c;
    int stride_a_batch, stride_b_batch, stride_c_batch;
    const void* sfa;
    const void* sfb;
    int stride_sfa, stride_sfb;
    int stride_sfa_batch, stride_sfb_batch;
    int scale_mode;      /* a8w8_scale_mode                                        */
    int c_dtype;         /* a8w8_c_dtype                                           */
    int b_preshuffled;   /* non-zero: b is in the a8w8_preshuffle_b layout (flatmm) */
} a8w8_gemm_args;

/* Dense GEMM, any scale mode.  Replaces the launch
 *   gemm_a8w8_blockscale_kernel<Traits><<<grid, 512>>>(kargs)   (host.cc:14-15, 249-257)
 * and the launches of the absent siblings gemm_a8w8_8wave (opus_gemm/rebuild.sh:3) for the
 * per-tensor and row/column modes.  Needs k % 128 == 0 and 16-byte aligned A/B rows for
 * the tiled kernels; other shapes run on a slower general kernel.  m, n edges are handled.
 * b_preshuffled != 0: B is in the a8w8_preshuffle_b layout (the weights a8w8_flatmm streams), so that one copy
 * of the weights serves prefill and decode; needs n % 16 == 0, k % 128 == 0 and 16-byte aligned pointers.
 * a16w16_gemm and a4w4_gemm accept it likewise for the weights their flat siblings stream (shuffled as bytes).
 * Skinny problems (m <= 128, n % 16 == 0, k % 64 == 0, 16-byte aligned rows; per-tensor, row/column, block or
 * tiled MX scales) run on the flat kernel of a8w8_flatmm where that is the faster one, on shuffled and on
 * row-major weights alike (a16w16_gemm and a4w4_gemm with tiled scales likewise). */
A8W8_API int a8w8_gemm(const a8w8_gemm_args* args, void* hip_stream);

/* The bf16 sibling (gemm_a16w16_8wave, the program opus_gemm/rebuild.sh:3-13 builds; its source is
 * absent from the reference): A [batch, m, k] and B [batch, n, k] hold bf16, C = A * B^T in bf16 or
 * fp32, fp32 accumulation, no scales (sfa, sfb, stride_sf*, scale_mode are ignored).  Runs on the
 * same pipelined kernel as a8w8_gemm with the 16x16x32 bf16 MFMA when k % 64 == 0, k >= 128 and rows
 * are 16-byte aligned; other shapes take a general kernel that follows the CPU order of operations. */
A8W8_API int a16w16_gemm(const a8w8_gemm_args* args, void* hip_stream);

/* The bf16 flat GEMM (flatmm_a16w16_gfx950, opus_fmm/README.md:10,51-57; source absent): A [batch, m, k]
 * bf16 with m <= 128, B bf16 pre-shuffled as a byte matrix -- a8w8_preshuffle_b[_device](b, out, n, 2*k) --
 * n % 16 == 0, k % 32 == 0, a, b and the rows of A 16-byte aligned, no scales, bf16 or fp32 C.  Same
 * streaming kernel as a8w8_flatmm. */
A8W8_API int a16w16_flatmm(const a8w8_gemm_args* args, void* hip_stream);

/* MXFP4 (OCP MX: E2M1 elements, two per byte with the even K index in the low nibble, one E8M0 scale per
 * 32 elements) through the same f8f6f4 instruction in its FP4 format (the reference names the format,
 * wmma_opus_rdna4/opus/opus.hpp:1854-1855, and has no program for it).  A [batch, m, k/2 bytes],
 * B [batch, n, k/2 bytes]; m, n, k and every stride count ELEMENTS (strides even); scale_mode is
 * MX_E8M0_1x32 (row-major scales, as a4w4_quantize_mx writes them by default) or MX_E8M0_TILED.  The MFMA kernels
 * take either when k % 256 == 0 and rows are 16-byte aligned (row-major scales: scale pointers and strides
 * multiples of 4; on the 128 x 128-tile kernel at any size, about half the rate of tiled scales on large problems);
 * everything else runs on the one-thread-per-element kernel. */
A8W8_API int a4w4_gemm(const a8w8_gemm_args* args, void* hip_stream);
/* MXFP4 skinny-M GEMM over pre-shuffled weights (no counterpart in the reference, which has neither an FP4
 * program nor a flat one for it; it is a8w8_flatmm for the FP4 form of the same instruction).  A [batch, m, k/2
 * bytes] with m <= 128; B pre-shuffled as the byte matrix it is -- a8w8_preshuffle_b[_device](b, out, n, k/2) --
 * with b_preshuffled != 0; sfa, sfb E8M0 in the MX_E8M0_TILED layout (a4w4_quantize_mx(tiled) or
 * a8w8_mx_tile_scales), scale_mode = MX_E8M0_TILED; n % 16 == 0, k % 128 == 0; m, n, k and the strides count
 * elements; a, b, sfa, sfb and the rows of A 16-byte aligned.  B is streamed once with 16-byte non-temporal loads. */
A8W8_API int a4w4_flatmm(const a8w8_gemm_args* args, void* hip_stream);
/* fp32 rows -> packed E2M1 + E8M0 scales: e = clamp(ceil(log2(amax32/6)), -127, 127), row-major scales
 * scale[r*(k/32) + p/32] or (tiled != 0) the MX_TILED layout. */
A8W8_API int a4w4_quantize_mx(const float* src_dev, int rows, int k, int ld, uint8_t* q_dev, uint8_t* scale_dev,
                              int tiled, void* hip_stream);

/* The block-scale entry point with exactly the reference's preconditions: scale_mode is
 * taken as BLOCK_1x128_128x128, n % 128 == 0 and k % 128 == 0 are required
 * (host.cc:179-187); c_dtype may be fp32 (the reference's output, common.h / host.cc:216)
 * or bf16. */
A8W8_API int a8w8_gemm_blockscale(const a8w8_gemm_args* args, void* hip_stream);

/* Skinny-M GEMM over pre-shuffled weights (the flatmm_a8w8_gfx950 program listed at
 * opus_fmm/README.md:9, built by opus_fmm/rebuild.sh:3-13).  Requires b_preshuffled != 0,
 * scale_mode ROWCOL, TENSOR, BLOCK_1x128_128x128 (scale arrays as for a8w8_gemm_blockscale; n, k % 128 == 0) or
 * MX_E8M0_TILED (MXFP8: both scale arrays in the tiled layout, 16-byte aligned),
 * m <= 128, n % 16 == 0, k % 64 == 0, a, b and the rows of A 16-byte aligned (A8W8_ERR_MISALIGNED otherwise).
 * B is streamed once, with 16-byte non-temporal loads, for up to 64 rows of A (twice, the second time from
 * cache, beyond).  Where a8w8_gemm's kernels are the
 * faster ones on the same shuffled weights (several groups of 16 rows over many short weight rows; k % 128 == 0
 * permitting) the call runs those, and a8w8_gemm with b_preshuffled takes this kernel for the skinny problems it
 * runs faster: either entry point gives the same kernel for the same problem. */
A8W8_API int a8w8_flatmm(const a8w8_gemm_args* args, void* hip_stream);

/* Host-side weight pre-shuffle, row-major b[n][k] -> Bshuf[n/16][k/64][4][16][16 bytes]:
 * byte (j, p) moves to ((j/16*(k/64) + p/64)*4 + (p%64)/16)*256 + (j%16)*16 + p%16.
 * The reference's own layout did not survive (source absent); this one is defined here.
 * a8w8_unshuffle_b is its inverse.  Both work on host memory. */
A8W8_API int a8w8_preshuffle_b(const void* b_host, void* out_host, int n, int k);
A8W8_API int a8w8_unshuffle_b(const void* bshuf_host, void* out_host, int n, int k);
/* The same permutation on device memory (src and dst must not overlap). */
A8W8_API int a8w8_preshuffle_b_device(const void* b_dev, void* out_dev, int n, int k, void* hip_stream);

/* fp32 -> E4M3, device buffers, one byte per element.
 *   clamp240 != 0: to_fp8_raw_from_fp32 (cvt_fp8/test.cpp:21-43): finite inputs are
 *       clamped to [-240, 240] by a median-of-three and then converted; NaN/Inf bypass the
 *       clamp and are converted as they are.
 *   clamp240 == 0: the unclamped packed convert of pk_cvt_fp8x4_fp32x4_rne
 *       (pk_cvt/test.cpp:220-257): elements 4i..4i+3 become the four bytes of word i,
 *       little-endian.
 * dialect OCP is the gfx950 hardware convert (the instruction both reference programs call by
 * builtin), round to nearest even and NOT saturating: NaN -> 0xFF, +-Inf -> 0x7F / 0xFF, and a
 * magnitude that rounds beyond 448 (anything above 464) -> the NaN code 0x7F | sign; so only
 * clamp240 protects against overflow.  Dialect FNUZ (bias 8, max 240, NaN 0x80, no -0: what
 * gfx942 hardware converts to) is computed in software on the device with the arithmetic of
 * ROCm's __hip_fp8_e4m3_fnuz: round to nearest even, saturating to +-240, NaN/Inf -> 0x80.
 * n == 0 is a no-op.  Returns an a8w8_status. */
A8W8_API int a8w8_cvt_f32_to_e4m3(const float* src_dev, uint8_t* dst_dev, size_t n, int dialect,
                                  int clamp240, void* hip_stream);
/* E4M3 -> fp32, device buffers: fp8_e4m3fnuz_to_fp32_raw (cvt_fp8/test.cpp:59-90) and
 * run_cast_from_f8<fp8, float, true> (pk_cvt/test.cpp:340-421) for FNUZ (0x80 -> NaN with
 * bits 0x7F800001); the hardware convert for OCP.  Returns an a8w8_status. */
A8W8_API int a8w8_cvt_e4m3_to_f32(const uint8_t* src_dev, float* dst_dev, size_t n, int dialect,
                                  void* hip_stream);

/* Quantisation front end: fp32 rows [rows, k] (leading dimension ld, elements) -> OCP E4M3
 * bytes [rows, k] plus scales, in the layouts a8w8_gemm consumes.
 *   ROWCOL: scale[r] = amax(row r)/448 (fp32)
 *   BLOCK : group_rows = 1   -> scale[(p/128)*rows + r]       (the SFA layout)
 *           group_rows = 128 -> scale[(r/128)*(k/128) + p/128] (the SFB layout)
 *   MX    : uint8 e = clamp(ceil(log2(amax32/448)), -127, 127) + 127 at scale[r*(k/32) + p/32]
 *   MX_TILED : the same bytes at their MX_TILED positions (a8w8_mx_tiled_bytes(rows, k) bytes)
 *   TENSOR: scale[0] = amax(all)/448 (four small launches; the scale slot holds the running amax
 *           in between, so it must not be read until the stream reaches the end of the call)
 * An all-zero group keeps scale 1 (E8M0 byte 0 for MX). */
A8W8_API int a8w8_quantize(const float* src_dev, int rows, int k, int ld, uint8_t* q_dev, void* scale_dev,
                           int scale_mode, int group_rows, void* hip_stream);

/* E8M0 scales, row-major sf[r*stride + k/32] -> the MX_TILED layout, device buffers
 * (a8w8_mx_tiled_bytes(rows, k) bytes at out, 16-byte aligned).  No counterpart in the
 * reference, which has no MXFP8 program; weights' scales are converted once, activations'
 * scales can be produced in this layout directly by a8w8_quantize. */
A8W8_API int a8w8_mx_tile_scales(const uint8_t* sf_dev, int rows, int k, int stride, uint8_t* out_dev,
                                 void* hip_stream);
/* Both scale arrays of one GEMM in a single launch (sfa [m][k/32] -> out_a, sfb [n][k/32] -> out_b). */
A8W8_API int a8w8_mx_tile_scales_ab(const uint8_t* sfa_dev, int m, int stride_sfa, uint8_t* out_a_dev,
                                    const uint8_t* sfb_dev, int n, int stride_sfb, uint8_t* out_b_dev, int k,
                                    void* hip_stream);
A8W8_API size_t a8w8_mx_tiled_bytes(int rows, int k);

/* Pre-processed weights on disk (host memory in, host memory out): the quantised B matrix, row-major
 * or in the a8w8_preshuffle_b layout, plus its scales in the layout a8w8_gemm / a8w8_flatmm read for
 * `scale_mode`, behind a 64-byte header, so that quantisation, shuffling and scale tiling are paid
 * once.  The reference keeps no such cache (its harness regenerates random weights per run).
 * File: header, n*k weight bytes, scale bytes (TENSOR 4; ROWCOL 4n; BLOCK 4*(n/128)*(k/128);
 * MX n*k/32; MX_TILED a8w8_mx_tiled_bytes(n, k)); `checksum` is FNV-1a-64 over both payloads. */
typedef struct {
    char magic[8];          /* "A8W8WGT" and a NUL                                  */
    uint32_t version;       /* 1                                                     */
    uint32_t n, k;
    uint32_t b_preshuffled; /* 0 row-major [n][k], 1 a8w8_preshuffle_b layout        */
    uint32_t scale_mode;    /* a8w8_scale_mode of the stored scales                  */
    uint32_t reserved;
    uint64_t b_bytes, scale_bytes;
    uint64_t checksum;
    uint64_t reserved2;
} a8w8_weight_header;

A8W8_API size_t a8w8_weight_scale_bytes(int n, int k, int scale_mode);
A8W8_API int a8w8_weights_save(const char* path, const void* b_host, const void* scale_host, int n, int k,
                               int b_preshuffled, int scale_mode);
/* Reads and checks the header only. */
A8W8_API int a8w8_weights_info(const char* path, a8w8_weight_header* out);
/* Reads both payloads into buffers of at least header.b_bytes / header.scale_bytes and verifies the checksum. */
A8W8_API int a8w8_weights_load(const char* path, void* b_host, size_t b_capacity, void* scale_host,
                               size_t scale_capacity);

A8W8_API const char* a8w8_status_string(int status);

/* Name of the kernel variant a8w8_gemm / a8w8_flatmm would launch for these arguments
 * (for logs and profiles); NULL if the arguments are rejected. */
A8W8_API const char* a8w8_kernel_name(const a8w8_gemm_args* args);

/* Measurement aid, not part of the GEMM path: reads `bytes` of device memory once with 16-byte non-temporal loads
 * from a grid sized to the machine and discards the values (`sink_dev`, 4 bytes, is never written for ordinary
 * data).  bytes / its launch time is the read bandwidth this device actually gives a streaming kernel -- the
 * yardstick beside the published HBM peak for a8w8_flatmm, after the reference's own
 * bandwidth_memread/bandwidth_kernel.cu:68-92.  bytes % 16 == 0, src_dev 16-byte aligned. */
A8W8_API int a8w8_hbm_read_probe(const void* src_dev, size_t bytes, void* sink_dev, void* hip_stream);

/* Measurement aid, no counterpart in the reference (its flat GEMM and its tile GEMM are separate programs): for a
 * skinny problem (m <= 128) both the flat kernel and the MFMA tile kernels can run, and the entry points choose
 * with a small cost model.  choice = A8W8_ROUTE_FLAT / A8W8_ROUTE_DENSE makes every later call in this process
 * take that side wherever both can run the problem, A8W8_ROUTE_MODEL (the default) restores the model.  For
 * timing the two sides against each other; a process-wide setting, not meant to be changed while other threads
 * are inside the library.  Returns the previous choice, or A8W8_ERR_BAD_MODE for an unknown one. */
enum { A8W8_ROUTE_MODEL = 0, A8W8_ROUTE_FLAT = 1, A8W8_ROUTE_DENSE = 2 };
A8W8_API int a8w8_route_override(int choice);

/* Optional explicit set-up of one device (device < 0: the current one): queries its architecture and
 * compute-unit count and raises the dynamic-LDS limit of every kernel variant.  The same work happens,
 * once per device and thread-safely, inside the first entry point called with that device current; call
 * this beforehand when that first call would otherwise fall inside a stream capture or a timed region.
 * No counterpart in the reference (its program configures nothing: one kernel, static LDS).
 * A8W8_OK, or A8W8_ERR_NO_DEVICE if the device is not a gfx950. */
A8W8_API int a8w8_init(int device);

/* Library version, major*10000 + minor*100 + patch. */
A8W8_API int a8w8_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MI355_A8W8_H */
