/*
 * CPU oracle for the A8W8 FP8 GEMM path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C restatement of the host-side arithmetic of
 * carlushuang/gcnasm for its FP8 GEMM demos.  It is linked only by the test
 * suite, the smoke check and the CPU-baseline leg of the benchmark; nothing
 * that ships in the product library may call it.
 *
 * Every function cites the reference file:line whose behaviour it restates
 * (paths relative to the reference checkout).
 *
 * Pinning status (what independent evidence fixes each function):
 *   orc_e4m3_fnuz_decode / orc_f8_cast_from_f8   two independent reference
 *       formulations (closed form vs bit manipulation) must agree on all 256
 *       codes; also fixed by the ROCm hip_fp8.h table fixture.
 *   orc_e4m3_ocp_decode    closed form of the OCP FP8 spec; hip_fp8.h fixture.
 *   orc_e4m3_*_encode      brute-force nearest-even over the decode table,
 *       hip_fp8.h fixture, known tie -54 -> -56 (cvt_fp8/test.cpp:133).
 *   orc_e4m3_ocp_encode_hw   the gfx950 hardware convert the reference calls by builtin
 *       (cvt_fp8/test.cpp:37, pk_cvt/test.cpp:242-243): the OCP FP8 specification's
 *       non-saturating conversion.  Equal to the saturating encoder wherever the rounded
 *       magnitude is representable (the hip_fp8.h fixture), overflow / Inf -> sign | 0x7F and
 *       NaN -> 0xFF as the specification's non-saturating mode prescribes; the GPU tests feed
 *       NaN, +-Inf, +-1e9, +-449, +-464, +-465 and +-241 to the instruction itself.
 *   orc_cvt_fp8_clamp240   the clamp is a median of three, the convert as above.
 *   orc_gemm_ref / orc_gemm_ref_mx   brute force in float64 on tiny shapes,
 *       exact-integer inputs, scale-mode reductions.
 *   orc_preshuffle_b       bijection + flatmm(A, shuffle(B)) == gemm(A, B).
 *   orc_gemm_bf16_ref      float64 matmul on small shapes, exact-integer inputs.
 *   orc_e2m1_* / orc_gemm_ref_mxfp4 / orc_quant_mxfp4   the OCP MX value table (16 codes, checked one by
 *       one), nearest-even against a brute force over the table, float64 matmul of the decoded
 *       operands, the quantiser's properties (largest element in (3, 6], error within half a step).
 *   orc_quant_*            no reference code (its harness has no quantiser): the recipe of the
 *       benchmark configurations, fixed by properties -- the group's largest element maps to
 *       +-448 (row/block) or into (224, 448] (MX, never saturating), dequantisation error within
 *       half an E4M3 ulp of every element, scale = amax/448 exactly, layouts as gemm_ref reads them.
 *   orc_mx_tile_scales     a layout this library defines (the reference has no MXFP8
 *       program): written as a walk over the layout's dimensions, i.e. the inverse of
 *       the index formula the kernels use; bijection on full blocks, padding = 127,
 *       and gemm(A, B, tile(sfa), tile(sfb)) == gemm(A, B, sfa, sfb).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* ------------------------------------------------------------------ decode */

/* E4M3 FNUZ (gfx942 dialect): bias 8, 0x80 = NaN, no infinities.
 * Restates fp8_e4m3fnuz_to_fp32_raw, cvt_fp8/test.cpp:59-90: sign/exponent/
 * mantissa split, exponent field 0 -> 0.mmm * 2^(1-bias), else 1.mmm * 2^(e-bias). */
ORC_API float orc_e4m3_fnuz_decode(uint8_t code)
{
    const int bias = 8;
    int s = (code >> 7) & 1, e = (code >> 3) & 0xf, m = code & 7;
    if (s == 1 && e == 0 && m == 0) return u2f(0x7fc00000u);
    float frac = (float)m / 8.0f;
    float v = (e == 0) ? frac * ldexpf(1.0f, 1 - bias) : (1.0f + frac) * ldexpf(1.0f, e - bias);
    return s ? -v : v;
}

/* Generic fp8 -> fp32 by bit manipulation.
 * Restates run_cast_from_f8<fp8_t, float, negative_zero_nan>, pk_cvt/test.cpp:340-421
 * with NumericUtils<fp8_t> (:316-327: exp 4, mant 3) and NumericUtils<float> (:281-296).
 * negative_zero_nan != 0: FNUZ (0x80 -> NaN bits 0x7F800001, bias 8).
 * negative_zero_nan == 0: the reference's "ieee mode": 0x80 -> -0, exponent field 15 ->
 * Inf (mantissa 0) or NaN, effective bias 7.  Returned as raw fp32 bits so that NaN
 * payloads can be compared exactly. */
ORC_API uint32_t orc_f8_cast_from_f8_bits(uint8_t x, int negative_zero_nan)
{
    const int in_exp = 4, in_mant = 3, out_exp = 8, out_mant = 23;
    const uint32_t Inf = 0x7F800000u, NegInf = 0xFF800000u, NaN = 0x7F800001u, Neg0 = 0x80000000u;
    if (x == 0) return 0;
    uint32_t sign = x >> (in_exp + in_mant);
    uint32_t mantissa = x & ((1u << in_mant) - 1);
    int exponent = (x & 0x7F) >> in_mant;
    const int exp_low_cutoff = (1 << (out_exp - 1)) - (1 << (in_exp - 1)) + 1 - (negative_zero_nan ? 1 : 0);
    if (negative_zero_nan) {
        if (x == 0x80) return NaN;
    } else {
        if (x == 0x80) return Neg0;
        if (exponent == ((1 << in_exp) - 1)) return (mantissa == 0) ? (sign ? NegInf : Inf) : NaN;
    }
    if (exponent == 0) { /* subnormal input: normalise (pk_cvt/test.cpp:400-407) */
        int sh = 1 + __builtin_clz(mantissa) - (32 - in_mant);
        mantissa <<= sh;
        exponent += 1 - sh;
        mantissa &= ((1u << in_mant) - 1);
    }
    exponent += exp_low_cutoff - 1;
    mantissa <<= out_mant - in_mant;
    if (exponent <= 0) { /* cannot happen for float output; kept for fidelity (:411-416) */
        mantissa |= 1u << out_mant;
        mantissa >>= 1 - exponent;
        exponent = 0;
    }
    return (sign << (out_exp + out_mant)) | ((uint32_t)exponent << out_mant) | mantissa;
}

/* E4M3 OCP ("E4M3FN", the dialect of __hip_fp8_e4m3 used at
 * opus_gemm/block_scale_gemm/gemm_a8w8_blockscale_host.cc:29,84 and of gfx950 hardware):
 * bias 7, 0x7F/0xFF = NaN, no infinities, max 448.  Closed form of the OCP FP8 spec. */
ORC_API float orc_e4m3_ocp_decode(uint8_t code)
{
    int s = (code >> 7) & 1, e = (code >> 3) & 0xf, m = code & 7;
    if (e == 15 && m == 7) return u2f(s ? 0xffc00000u : 0x7fc00000u);
    float frac = (float)m / 8.0f;
    float v = (e == 0) ? frac * ldexpf(1.0f, -6) : (1.0f + frac) * ldexpf(1.0f, e - 7);
    return s ? -v : v;
}

/* E8M0 shared exponent (OCP MX): 2^(b-127), 255 = NaN.  Matches the scaled-MFMA scale
 * operand contract noted at wmma_opus_rdna4/opus/opus.hpp:1786 (127 is the identity). */
ORC_API float orc_e8m0_decode(uint8_t b)
{
    if (b == 255) return u2f(0x7fc00000u);
    return ldexpf(1.0f, (int)b - 127);
}

/* ------------------------------------------------------------------ encode */

/* fp32 -> E4M3 with round-to-nearest-even and saturation to the largest finite value.
 * Semantics of static_cast<__hip_fp8_e4m3>(float) (gemm_a8w8_blockscale_host.cc:41) for
 * fnuz == 0 and of the gfx942 hardware convert (cvt_fp8/test.cpp:37) for fnuz != 0:
 *   NaN or Inf  -> NaN code (0x7F | sign for OCP, 0x80 for FNUZ)
 *   |x| > max   -> +-max (0x7E / 0x7F | sign)
 * Own formulation: scale the magnitude to an integer number of quanta and round it with
 * nearbyintf in the default (nearest-even) mode. */
static uint8_t encode_e4m3(float x, int fnuz)
{
    const int bias = fnuz ? 8 : 7;
    const float fmax = fnuz ? 240.0f : 448.0f;
    const uint8_t max_code = fnuz ? 0x7f : 0x7e;
    uint32_t u = f2u(x);
    uint8_t sign = (uint8_t)((u >> 31) << 7);
    if ((u & 0x7F800000u) == 0x7F800000u) return fnuz ? 0x80 : (uint8_t)(sign | 0x7f);
    float ax = fabsf(x);
    if (ax > fmax) return (uint8_t)(sign | max_code);
    if (ax == 0.0f) return fnuz ? 0 : sign;
    int e;
    (void)frexpf(ax, &e); /* ax = f * 2^e, f in [0.5, 1) -> unbiased exponent e-1 */
    int ue = e - 1;
    int emin = 1 - bias;            /* exponent of the smallest normal */
    if (ue < emin) ue = emin;       /* subnormal range shares the smallest normal's quantum */
    float q = nearbyintf(ldexpf(ax, 3 - ue)); /* quanta of 2^(ue-3); 8..16 for normals */
    if (q >= 16.0f) { q = 8.0f; ue += 1; }
    int qi = (int)q;
    uint8_t code;
    if (qi < 8) code = (uint8_t)qi;                       /* subnormal (or zero) */
    else code = (uint8_t)(((ue + bias) << 3) | (qi - 8));
    if (code > max_code) code = max_code;                 /* unreachable after the clip above */
    if (fnuz && code == 0) return 0;                      /* FNUZ has no negative zero */
    return (uint8_t)(sign | code);
}

ORC_API uint8_t orc_e4m3_ocp_encode(float x) { return encode_e4m3(x, 0); }
ORC_API uint8_t orc_e4m3_fnuz_encode(float x) { return encode_e4m3(x, 1); }

/* What __builtin_amdgcn_cvt_pk_fp8_f32 returns on gfx950 (the instruction behind
 * cvt_fp8/test.cpp:37 and pk_cvt/test.cpp:242-243 on this target): OCP E4M3, round to nearest
 * even, NOT saturating -- the non-saturating conversion of the OCP FP8 specification:
 *   NaN (either sign)                  -> 0xFF
 *   +-Inf                              -> sign | 0x7F   (the NaN code: E4M3 has no infinity)
 *   magnitude that rounds beyond 448   -> sign | 0x7F   (everything above the tie 464;
 *                                         (448, 464] still rounds to 448 = 0x7E)
 *   everything else                    as the saturating encoder above. */
ORC_API uint8_t orc_e4m3_ocp_encode_hw(float x)
{
    const uint32_t u = f2u(x);
    const uint8_t sign = (uint8_t)((u >> 31) << 7);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0xff;
    if (fabsf(x) > 464.0f) return (uint8_t)(sign | 0x7f);      /* includes +-Inf */
    return encode_e4m3(x, 0);
}
/* The convert of dialect `fnuz`: the gfx950 instruction for OCP; for FNUZ the conversion of ROCm's
 * __hip_fp8_e4m3_fnuz (round to nearest even, saturating to +-240, NaN/Inf -> 0x80), which is what
 * the library computes in software for that dialect. */
static uint8_t convert_e4m3(float x, int fnuz) { return fnuz ? encode_e4m3(x, 1) : orc_e4m3_ocp_encode_hw(x); }

/* to_fp8_raw_from_fp32, cvt_fp8/test.cpp:21-43: unless the input is NaN/Inf it is clamped
 * to [-240, 240] with a median-of-three, then converted by the hardware instruction in
 * the dialect of the target (fnuz != 0: gfx942, fnuz == 0: gfx950 / OCP).  NaN/Inf inputs
 * bypass the clamp and go through the convert as they are: on gfx950 NaN -> 0xFF,
 * +Inf -> 0x7F, -Inf -> 0xFF; FNUZ 0x80 for all three. */
ORC_API uint8_t orc_cvt_fp8_clamp240(float v, int fnuz)
{
    uint32_t u = f2u(v);
    if ((u & 0x7F800000u) != 0x7F800000u) {
        if (v > 240.0f) v = 240.0f;
        if (v < -240.0f) v = -240.0f;
    }
    return convert_e4m3(v, fnuz);
}

/* pk_cvt_fp8x4_fp32x4_rne, pk_cvt/test.cpp:220-257: two packed converts (s0,s1)->x and
 * (s2,s3)->y, both into the low word, then a byte permute with selector 0x05040100 that
 * yields bytes [x.b0, x.b1, y.b0, y.b1], i.e. little-endian [f8(s0), f8(s1), f8(s2), f8(s3)].
 * No clamp is applied before the convert, so on gfx950 magnitudes that round beyond 448 come out
 * as the NaN code (orc_e4m3_ocp_encode_hw). */
ORC_API uint32_t orc_pk_cvt_fp8x4(const float s[4], int fnuz)
{
    uint32_t x = (uint32_t)convert_e4m3(s[0], fnuz) | ((uint32_t)convert_e4m3(s[1], fnuz) << 8);
    uint32_t y = (uint32_t)convert_e4m3(s[2], fnuz) | ((uint32_t)convert_e4m3(s[3], fnuz) << 8);
    /* v_perm_b32(y, x, 0x05040100): selector bytes 0,1 pick x.b0,x.b1; 4,5 pick y.b0,y.b1 */
    return (x & 0xffffu) | ((y & 0xffffu) << 16);
}

/* fp32 -> bf16, round to nearest even (bits += 0x7FFF + lsb), NaN kept quiet.
 * Formula as at wmma_opus_rdna4/opus/opus.hpp:944-950. */
ORC_API uint16_t orc_f32_to_bf16(float f)
{
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
ORC_API float orc_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* vector forms used by the tests */
ORC_API void orc_decode_vec(const uint8_t* in, float* out, size_t n, int dialect)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = dialect == 0 ? orc_e4m3_ocp_decode(in[i]) : orc_e4m3_fnuz_decode(in[i]);
}
ORC_API void orc_encode_vec(const float* in, uint8_t* out, size_t n, int dialect, int clamp240)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i)
        out[i] = clamp240 ? orc_cvt_fp8_clamp240(in[i], dialect) : encode_e4m3(in[i], dialect);
}
/* the unclamped convert of the device (pk_cvt_fp8x4_fp32x4_rne element by element) */
ORC_API void orc_convert_vec(const float* in, uint8_t* out, size_t n, int dialect)
{
    for (size_t i = 0; i < n; ++i) out[i] = convert_e4m3(in[i], dialect);
}
ORC_API void orc_bf16_vec(const float* in, uint16_t* out, size_t n)
{
    for (size_t i = 0; i < n; ++i) out[i] = orc_f32_to_bf16(in[i]);
}

/* -------------------------------------------------------------------- GEMM */

static float lut_ocp[256];
static int lut_ready;
static void init_lut(void)
{
    if (lut_ready) return;
    for (int i = 0; i < 256; ++i) lut_ocp[i] = orc_e4m3_ocp_decode((uint8_t)i);
    lut_ready = 1;
}

/* gemm_ref, gemm_a8w8_blockscale_host.cc:66-90, same argument list and index formulas:
 *   C[i,j] = sum over k-groups g, p in g:  float(A[i,p]) * float(B[j,p]) * (sfa * sfb)
 *   sfa = SFA[g*stride_sfa + i/group_m],  sfb = SFB[(j/group_n)*stride_sfb + g]
 * sequential p, fp32 accumulation, one product-times-scale per MAC (host.cc:84).
 * The scale modes of the library map onto it as
 *   per-tensor  group_m=M, group_n=N, group_k=K, strides 0
 *   row/col     group_m=1, group_n=1, group_k=K, stride_sfa=0, stride_sfb=1
 *   1x128/128x128 block   group_m=1, group_n=128, group_k=128 (host.cc:244-245)
 * rows [row_begin,row_end) only, so that large problems can be checked on a slab.
 * decode_per_mac != 0 keeps the reference's two software decodes per MAC (that is where
 * its time goes and what the CPU baseline times); 0 uses a 256-entry table, same values. */
ORC_API void orc_gemm_ref(const uint8_t* a, const uint8_t* b, const float* sfa, const float* sfb,
                          float* c, int m, int n, int k, int lda, int ldb, int ldc,
                          int stride_sfa, int stride_sfb, int group_m, int group_n, int group_k,
                          int row_begin, int row_end, int decode_per_mac)
{
    init_lut();
    (void)m;
#pragma omp parallel for collapse(2) schedule(static)
    for (int i = row_begin; i < row_end; ++i) {
        for (int j = 0; j < n; ++j) {
            const uint8_t* a_row = a + (size_t)i * lda;
            const uint8_t* b_row = b + (size_t)j * ldb;
            const int m_group = i / group_m, n_group = j / group_n;
            float sum = 0.0f;
            for (int g = 0; g < k / group_k; ++g) {
                const float scale = sfa[(size_t)g * stride_sfa + m_group] * sfb[(size_t)n_group * stride_sfb + g];
                const int p0 = g * group_k, p1 = p0 + group_k;
                if (decode_per_mac) {
                    for (int p = p0; p < p1; ++p)
                        sum += orc_e4m3_ocp_decode(a_row[p]) * orc_e4m3_ocp_decode(b_row[p]) * scale;
                } else {
                    for (int p = p0; p < p1; ++p) sum += lut_ocp[a_row[p]] * lut_ocp[b_row[p]] * scale;
                }
            }
            c[(size_t)i * ldc + j] = sum;
        }
    }
}

/* MXFP8 GEMM: gemm_ref with group_k = 32, group_m = group_n = 1 and E8M0 scales laid out
 * K-contiguous per row: ea[i*stride_sfa + p/32], eb[j*stride_sfb + p/32].  The scale of a
 * MAC is 2^(ea-127) * 2^(eb-127), formed as one exact ldexp so that it cannot over/underflow
 * halfway.  No harness for this mode exists in the reference; the math is gemm_ref's
 * (host.cc:66-90) with the scale decode of opus.hpp:1786. */
ORC_API void orc_gemm_ref_mx(const uint8_t* a, const uint8_t* b, const uint8_t* ea, const uint8_t* eb,
                             float* c, int m, int n, int k, int lda, int ldb, int ldc,
                             int stride_sfa, int stride_sfb, int row_begin, int row_end, int decode_per_mac)
{
    init_lut();
    (void)m;
#pragma omp parallel for collapse(2) schedule(static)
    for (int i = row_begin; i < row_end; ++i) {
        for (int j = 0; j < n; ++j) {
            const uint8_t* a_row = a + (size_t)i * lda;
            const uint8_t* b_row = b + (size_t)j * ldb;
            float sum = 0.0f;
            for (int g = 0; g < k / 32; ++g) {
                uint8_t xa = ea[(size_t)i * stride_sfa + g], xb = eb[(size_t)j * stride_sfb + g];
                float scale = (xa == 255 || xb == 255) ? u2f(0x7fc00000u)
                                                       : ldexpf(1.0f, (int)xa + (int)xb - 254);
                if (decode_per_mac) {
                    for (int p = g * 32; p < g * 32 + 32; ++p)
                        sum += orc_e4m3_ocp_decode(a_row[p]) * orc_e4m3_ocp_decode(b_row[p]) * scale;
                } else {
                    for (int p = g * 32; p < g * 32 + 32; ++p) sum += lut_ocp[a_row[p]] * lut_ocp[b_row[p]] * scale;
                }
            }
            c[(size_t)i * ldc + j] = sum;
        }
    }
}

/* ------------------------------------------------------------ MXFP4 (OCP MX, E2M1 elements)
 * The reference stops at naming the instruction's FP4 format (wmma_opus_rdna4/opus/opus.hpp:1854-1855);
 * arithmetic per the OCP Microscaling spec v1.0: E2M1 = sign, 2 exponent bits (bias 1), 1 mantissa bit,
 * values +-{0, 0.5, 1, 1.5, 2, 3, 4, 6}, no NaN / infinity; two elements per byte, the even K index in
 * the low nibble; one E8M0 scale per 32 elements. */
static const float e2m1_values[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
ORC_API float orc_e2m1_decode(uint8_t nibble)
{
    const float v = e2m1_values[nibble & 7];
    return (nibble & 8) ? -v : v;
}
/* round to nearest, ties to the value with an even mantissa bit, saturating at +-6 */
ORC_API uint8_t orc_e2m1_encode(float x)
{
    const uint8_t sign = signbit(x) ? 8 : 0;
    const float a = fabsf(x);
    if (!(a == a)) return (uint8_t)(sign | 7);              /* NaN has no code: saturate */
    int best = 0;
    for (int c = 1; c < 8; ++c) {
        const float d0 = fabsf(a - e2m1_values[best]), d1 = fabsf(a - e2m1_values[c]);
        if (d1 < d0 || (d1 == d0 && (c & 1) == 0)) best = c;
    }
    return (uint8_t)(sign | best);
}
static inline float fp4_at(const uint8_t* row, int p) { return orc_e2m1_decode((uint8_t)((row[p >> 1] >> ((p & 1) * 4)) & 15)); }

/* C = A * B^T for packed E2M1 A [m][k/2], B [n][k/2] and E8M0 scales [rows][k/32]: gemm_ref's loop
 * (host.cc:66-90) with group_k = 32 and scale = 2^(ea-127) * 2^(eb-127). */
ORC_API void orc_gemm_ref_mxfp4(const uint8_t* a, const uint8_t* b, const uint8_t* ea, const uint8_t* eb, float* c,
                                int m, int n, int k, int row_begin, int row_end)
{
    (void)m;
#pragma omp parallel for collapse(2) schedule(static)
    for (int i = row_begin; i < row_end; ++i)
        for (int j = 0; j < n; ++j) {
            const uint8_t* a_row = a + (size_t)i * (k / 2);
            const uint8_t* b_row = b + (size_t)j * (k / 2);
            float sum = 0.0f;
            for (int g = 0; g < k / 32; ++g) {
                const uint8_t xa = ea[(size_t)i * (k / 32) + g], xb = eb[(size_t)j * (k / 32) + g];
                const float scale = (xa == 255 || xb == 255) ? u2f(0x7fc00000u) : ldexpf(1.0f, (int)xa + (int)xb - 254);
                for (int p = g * 32; p < g * 32 + 32; ++p) sum += fp4_at(a_row, p) * fp4_at(b_row, p) * scale;
            }
            c[(size_t)i * n + j] = sum;
        }
}

/* MXFP4 quantiser: e = clamp(ceil(log2(amax/6)), -127, 127), byte e + 127, q = E2M1(x * 2^-e): the
 * ceiling keeps the largest element at or below 6. */
ORC_API void orc_quant_mxfp4(const float* x, int rows, int k, int ld, uint8_t* q, uint8_t* scale)
{
    for (int r = 0; r < rows; ++r)
        for (int g = 0; g < k / 32; ++g) {
            float amax = 0.0f;
            for (int p = 0; p < 32; ++p) amax = fmaxf(amax, fabsf(x[(size_t)r * ld + g * 32 + p]));
            const float t = amax / 6.0f;
            int e = -127;
            if (t > 0.0f) {
                e = ilogbf(t);
                if (t > ldexpf(1.0f, e)) ++e;
                if (e < -127) e = -127;
                if (e > 127) e = 127;
            }
            scale[(size_t)r * (k / 32) + g] = (uint8_t)(e + 127);
            for (int p = 0; p < 32; p += 2) {
                const uint8_t lo = orc_e2m1_encode(ldexpf(x[(size_t)r * ld + g * 32 + p], -e));
                const uint8_t hi = orc_e2m1_encode(ldexpf(x[(size_t)r * ld + g * 32 + p + 1], -e));
                q[(size_t)r * (k / 2) + (g * 32 + p) / 2] = (uint8_t)(lo | (hi << 4));
            }
        }
}

/* Selected (i,j) probes of either GEMM, for spot checks at sizes where a slab is too slow.
 * mode 3 = MX (sfa/sfb are uint8), else fp32 scales with the gemm_ref grouping. */
ORC_API void orc_gemm_probe(const uint8_t* a, const uint8_t* b, const void* sfa, const void* sfb,
                            int k, int lda, int ldb, int stride_sfa, int stride_sfb,
                            int group_m, int group_n, int group_k, int mode,
                            const int* pi, const int* pj, int nprobe, float* out)
{
    init_lut();
#pragma omp parallel for schedule(static)
    for (int t = 0; t < nprobe; ++t) {
        int i = pi[t], j = pj[t];
        const uint8_t* a_row = a + (size_t)i * lda;
        const uint8_t* b_row = b + (size_t)j * ldb;
        float sum = 0.0f;
        if (mode == 3) {
            const uint8_t *ea = sfa, *eb = sfb;
            for (int g = 0; g < k / 32; ++g) {
                uint8_t xa = ea[(size_t)i * stride_sfa + g], xb = eb[(size_t)j * stride_sfb + g];
                float scale = (xa == 255 || xb == 255) ? u2f(0x7fc00000u)
                                                       : ldexpf(1.0f, (int)xa + (int)xb - 254);
                for (int p = g * 32; p < g * 32 + 32; ++p) sum += lut_ocp[a_row[p]] * lut_ocp[b_row[p]] * scale;
            }
        } else {
            const float *fa = sfa, *fb = sfb;
            for (int g = 0; g < k / group_k; ++g) {
                float scale = fa[(size_t)g * stride_sfa + i / group_m] * fb[(size_t)(j / group_n) * stride_sfb + g];
                for (int p = g * group_k; p < (g + 1) * group_k; ++p)
                    sum += lut_ocp[a_row[p]] * lut_ocp[b_row[p]] * scale;
            }
        }
        out[t] = sum;
    }
}

/* ------------------------------------------------------------------ flatmm */

/* Weight pre-shuffle for the skinny-M path.  The reference source that defined its layout
 * (opus_fmm/flatmm_a8w8_gfx950.cc, listed at opus_fmm/README.md:9) is absent, so the
 * layout is this library's own:
 *     Bshuf[N/16][K/64][kq = 4][n = 16][16 bytes]
 * i.e. byte (n, k) of row-major B[N][K] moves to
 *     ((n/16 * (K/64) + k/64) * 4 + (k%64)/16) * 256 + (n%16) * 16 + k%16.
 * One 64-lane load of 16 bytes per lane then covers 16 rows x 64 K contiguously (1 KiB)
 * with lane = kq*16 + n, the operand order of the 16x16 FP8 MFMA. */
ORC_API size_t orc_preshuffle_index(int n, int k, int K)
{
    return (((size_t)(n / 16) * (K / 64) + k / 64) * 4 + (k % 64) / 16) * 256 + (size_t)(n % 16) * 16 + k % 16;
}
ORC_API void orc_preshuffle_b(const uint8_t* b, uint8_t* out, int N, int K)
{
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k) out[orc_preshuffle_index(n, k, K)] = b[(size_t)n * K + k];
}
ORC_API void orc_unshuffle_b(const uint8_t* bs, uint8_t* out, int N, int K)
{
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k) out[(size_t)n * K + k] = bs[orc_preshuffle_index(n, k, K)];
}

/* Tiled layout of MX E8M0 scales (defined by this library; no reference counterpart).
 * Dimensions, outermost first, one byte per innermost element:
 *     [K/512][ceil(rows/64)][pair of K steps: 2][r16: 16][g: 4][jp: 2][par: 2][s: 2]
 * holding the exponent of row  64*blk + 32*jp + 8*(r16/4) + 4*par + r16%4  and of 32-wide
 * K block  16*kg + 8*pair + 4*s + g.  Rows past `rows` and blocks past k/32 hold 127. */
ORC_API size_t orc_mx_tiled_bytes(int rows, int k)
{
    return (size_t)((k + 511) / 512) * (size_t)((rows + 63) / 64) * 1024;
}
ORC_API void orc_mx_tile_scales(const uint8_t* sf, int rows, int k, int stride, uint8_t* out)
{
    const int groups = (k + 511) / 512, nblk = (rows + 63) / 64, blocks = k / 32;
    uint8_t* o = out;
    for (int kg = 0; kg < groups; ++kg)
        for (int blk = 0; blk < nblk; ++blk)
            for (int pair = 0; pair < 2; ++pair)
                for (int r16 = 0; r16 < 16; ++r16)
                    for (int g = 0; g < 4; ++g)
                        for (int jp = 0; jp < 2; ++jp)
                            for (int par = 0; par < 2; ++par)
                                for (int st = 0; st < 2; ++st) {
                                    const int row = 64 * blk + 32 * jp + 8 * (r16 / 4) + 4 * par + r16 % 4;
                                    const int kblk = 16 * kg + 8 * pair + 4 * st + g;
                                    *o++ = (row < rows && kblk < blocks) ? sf[(size_t)row * stride + kblk] : 127;
                                }
}
ORC_API void orc_mx_untile_scales(const uint8_t* tiled, int rows, int k, int stride, uint8_t* sf)
{
    const int groups = (k + 511) / 512, nblk = (rows + 63) / 64, blocks = k / 32;
    const uint8_t* o = tiled;
    for (int kg = 0; kg < groups; ++kg)
        for (int blk = 0; blk < nblk; ++blk)
            for (int pair = 0; pair < 2; ++pair)
                for (int r16 = 0; r16 < 16; ++r16)
                    for (int g = 0; g < 4; ++g)
                        for (int jp = 0; jp < 2; ++jp)
                            for (int par = 0; par < 2; ++par)
                                for (int st = 0; st < 2; ++st, ++o) {
                                    const int row = 64 * blk + 32 * jp + 8 * (r16 / 4) + 4 * par + r16 % 4;
                                    const int kblk = 16 * kg + 8 * pair + 4 * st + g;
                                    if (row < rows && kblk < blocks) sf[(size_t)row * stride + kblk] = *o;
                                }
}

/* flatmm oracle that consumes the SHUFFLED weights directly: gemm_ref's math
 * (host.cc:66-90) with per-row A scale and per-row B scale applied per MAC. */
ORC_API void orc_flatmm_ref(const uint8_t* a, const uint8_t* bshuf, const float* sfa, const float* sfb,
                            float* c, int m, int n, int k, int lda, int ldc)
{
    init_lut();
#pragma omp parallel for collapse(2) schedule(static)
    for (int i = 0; i < m; ++i) {
        for (int j = 0; j < n; ++j) {
            float sum = 0.0f;
            const float scale = sfa[i] * sfb[j];
            for (int p = 0; p < k; ++p)
                sum += lut_ocp[a[(size_t)i * lda + p]] * lut_ocp[bshuf[orc_preshuffle_index(j, p, k)]] * scale;
            c[(size_t)i * ldc + j] = sum;
        }
    }
}

/* bf16 x bf16 GEMM of the a16w16 sibling (its source is absent; opus_gemm/rebuild.sh:3 names it): the same
 * loop as gemm_ref, host.cc:66-90, without scales -- fp32 accumulation over K in order, C[i][j] =
 * sum_k float(A[i][k]) * float(B[j][k]).  a, b hold bf16 bit patterns. */
ORC_API void orc_gemm_bf16_ref(const uint16_t* a, const uint16_t* b, float* c, int m, int n, int k, int lda, int ldb,
                               int ldc)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            float sum = 0.0f;
            for (int p = 0; p < k; ++p)
                sum += u2f((uint32_t)a[(size_t)i * lda + p] << 16) * u2f((uint32_t)b[(size_t)j * ldb + p] << 16);
            c[(size_t)i * ldc + j] = sum;
        }
}

/* ------------------------------------------------------------ quantisation front end
 * The recipe the benchmark configurations state: scale = amax(group)/448, q = E4M3-OCP(x / scale)
 * with round-to-nearest-even and saturation; group = a row (per token / per channel), a 1 x 128
 * block (A-side block scales, stored [k/128][rows] as gemm_a8w8_blockscale_host.cc:78 indexes
 * them) or a 128 x 128 block (B side, stored [rows/128][k/128], host.cc:79).  The reference has no
 * quantiser (its harness casts uniform random floats, host.cc:32-44); an all-zero group keeps
 * scale 1 so that it dequantises to zeros instead of 0/0. */
static float group_scale(float amax) { return amax > 0.0f ? amax / 448.0f : 1.0f; }

ORC_API void orc_quant_rowwise(const float* x, int rows, int k, int ld, uint8_t* q, float* scale)
{
    for (int r = 0; r < rows; ++r) {
        float amax = 0.0f;
        for (int p = 0; p < k; ++p) amax = fmaxf(amax, fabsf(x[(size_t)r * ld + p]));
        const float s = group_scale(amax);
        scale[r] = s;
        for (int p = 0; p < k; ++p) q[(size_t)r * k + p] = orc_e4m3_ocp_encode(x[(size_t)r * ld + p] / s);
    }
}

ORC_API void orc_quant_tensor(const float* x, int rows, int k, int ld, uint8_t* q, float* scale)
{
    float amax = 0.0f;
    for (int r = 0; r < rows; ++r)
        for (int p = 0; p < k; ++p) amax = fmaxf(amax, fabsf(x[(size_t)r * ld + p]));
    const float s = group_scale(amax);
    scale[0] = s;
    for (int r = 0; r < rows; ++r)
        for (int p = 0; p < k; ++p) q[(size_t)r * k + p] = orc_e4m3_ocp_encode(x[(size_t)r * ld + p] / s);
}

ORC_API void orc_quant_block(const float* x, int rows, int k, int ld, uint8_t* q, float* scale, int group_rows)
{
    const int gk = k / 128;
    for (int r0 = 0; r0 < rows; r0 += group_rows)
        for (int g = 0; g < gk; ++g) {
            float amax = 0.0f;
            for (int r = r0; r < r0 + group_rows; ++r)
                for (int p = 0; p < 128; ++p) amax = fmaxf(amax, fabsf(x[(size_t)r * ld + g * 128 + p]));
            const float s = group_scale(amax);
            if (group_rows == 1) scale[(size_t)g * rows + r0] = s;
            else scale[(size_t)(r0 / group_rows) * gk + g] = s;
            for (int r = r0; r < r0 + group_rows; ++r)
                for (int p = 0; p < 128; ++p)
                    q[(size_t)r * k + g * 128 + p] = orc_e4m3_ocp_encode(x[(size_t)r * ld + g * 128 + p] / s);
        }
}

/* MX: e = clamp(ceil(log2(amax/448)), -127, 127), byte e + 127, q = E4M3-OCP(x * 2^-e).  The ceiling
 * means the largest element never saturates (|x| 2^-e <= 448).  ceil(log2 t) is taken exactly:
 * the binary exponent of t, plus one unless t is a power of two. */
ORC_API void orc_quant_mx(const float* x, int rows, int k, int ld, uint8_t* q, uint8_t* scale)
{
    for (int r = 0; r < rows; ++r)
        for (int g = 0; g < k / 32; ++g) {
            float amax = 0.0f;
            for (int p = 0; p < 32; ++p) amax = fmaxf(amax, fabsf(x[(size_t)r * ld + g * 32 + p]));
            const float t = amax / 448.0f;
            int e = -127;
            if (t > 0.0f) {
                e = ilogbf(t);
                if (t > ldexpf(1.0f, e)) ++e;
                if (e < -127) e = -127;
                if (e > 127) e = 127;
            }
            scale[(size_t)r * (k / 32) + g] = (uint8_t)(e + 127);
            for (int p = 0; p < 32; ++p)
                q[(size_t)r * k + g * 32 + p] = orc_e4m3_ocp_encode(ldexpf(x[(size_t)r * ld + g * 32 + p], -e));
        }
}

/* valid_vector, gemm_a8w8_blockscale_host.cc:46-63: count of elements whose absolute
 * difference exceeds the threshold (the reference stops at 10; the full count is returned). */
ORC_API long orc_count_abs_mismatch(const float* ref, const float* out, size_t n, float thr)
{
    long bad = 0;
    for (size_t i = 0; i < n; ++i)
        if (!(fabsf(ref[i] - out[i]) <= thr)) ++bad;
    return bad;
}

ORC_API int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
