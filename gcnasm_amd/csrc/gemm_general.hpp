// General-shape A8W8 GEMM for gfx950: any m, n, k, strides and alignment, every scale mode.
// One thread per element of C, sequential K, one product-times-scale per MAC without fused
// multiply-add, i.e. the arithmetic order of the reference CPU GEMM
// (opus_gemm/block_scale_gemm/gemm_a8w8_blockscale_host.cc:66-90).  It is the path for
// shapes the tiled kernels do not take (k % 128 != 0, unaligned rows); it is not fast.
#pragma once
#include "a8w8_device.hpp"

namespace a8w8 {

A8W8_DEV float e4m3_to_f32_hw(uint8_t code) { return __builtin_amdgcn_cvt_f32_fp8((int)code, 0); }

A8W8_DEV float e8m0_pair_scale(uint8_t ea, uint8_t eb)
{
    if (ea == 255 || eb == 255) return __builtin_nanf("");
    return __builtin_ldexpf(1.0f, (int)ea + (int)eb - 254);
}

template <int MODE, int CDT>
__global__ void __launch_bounds__(256) gemm_a8w8_general(GemmParams p)
{
#pragma clang fp contract(off)   // separate multiply and add, as the reference's host code rounds
    const int j = blockIdx.x * 16 + (threadIdx.x & 15);
    const int i = blockIdx.y * 16 + (threadIdx.x >> 4);
    const int batch = blockIdx.z;
    if (i >= p.m || j >= p.n) return;
    const uint8_t* a = p.a + (long long)batch * p.a_batch + (long long)i * p.lda;
    const uint8_t* b = p.b + (long long)batch * p.b_batch + (long long)j * p.ldb;
    const float* sfa_f = (const float*)p.sfa + (long long)batch * p.sfa_batch;
    const float* sfb_f = (const float*)p.sfb + (long long)batch * p.sfb_batch;
    const uint8_t* sfa_e = (const uint8_t*)p.sfa + (long long)batch * p.sfa_batch;
    const uint8_t* sfb_e = (const uint8_t*)p.sfb + (long long)batch * p.sfb_batch;

    const int group_k = MODE == MODE_BLOCK ? 128 : ((MODE == MODE_MX || MODE == MODE_MXT) ? 32 : p.k);
    float sum = 0.f;
    for (int k0 = 0; k0 < p.k; k0 += group_k) {
        const int g = k0 / group_k;
        float scale;
        if constexpr (MODE == MODE_TENSOR) scale = sfa_f[0] * sfb_f[0];
        if constexpr (MODE == MODE_ROWCOL) scale = sfa_f[i] * sfb_f[j];
        if constexpr (MODE == MODE_BLOCK)
            scale = sfa_f[(long long)g * p.stride_sfa + i] * sfb_f[(long long)(j >> 7) * p.stride_sfb + g];
        if constexpr (MODE == MODE_MX)
            scale = e8m0_pair_scale(sfa_e[(long long)i * p.stride_sfa + g], sfb_e[(long long)j * p.stride_sfb + g]);
        if constexpr (MODE == MODE_MXT)
            scale = e8m0_pair_scale(sfa_e[mx_tiled_index(p.m, i, g)], sfb_e[mx_tiled_index(p.n, j, g)]);
        const int k1 = min(k0 + group_k, p.k);
        for (int k = k0; k < k1; ++k) {
            const float prod = e4m3_to_f32_hw(a[k]) * e4m3_to_f32_hw(b[k]);
            const float term = prod * scale;
            sum = sum + term;
        }
    }
    const long long ci = (long long)batch * p.c_batch + (long long)i * p.ldc + j;
    if constexpr (CDT == C_BF16) ((unsigned short*)p.c)[ci] = bf16_bits(sum);
    else ((float*)p.c)[ci] = sum;
}

// bf16 x bf16 -> fp32 accumulate, any shape: the order of operations of the reference CPU GEMM
// (sequential K, product then add, no fused multiply-add).  a, b hold bf16 bit patterns.
template <int CDT>
__global__ void __launch_bounds__(256) gemm_a16w16_general(const unsigned short* a, const unsigned short* b, void* c, int m, int n,
                                                           int k, int lda, int ldb, int ldc, long long a_batch, long long b_batch,
                                                           long long c_batch)
{
#pragma clang fp contract(off)
    const int j = blockIdx.x * 16 + (threadIdx.x & 15);
    const int i = blockIdx.y * 16 + (threadIdx.x >> 4);
    const int batch = blockIdx.z;
    if (i >= m || j >= n) return;
    const unsigned short* ar = a + batch * a_batch + (long long)i * lda;
    const unsigned short* br = b + batch * b_batch + (long long)j * ldb;
    float sum = 0.f;
    for (int p = 0; p < k; ++p) {
        const float prod = __uint_as_float((unsigned)ar[p] << 16) * __uint_as_float((unsigned)br[p] << 16);
        sum = sum + prod;
    }
    const long long ci = batch * c_batch + (long long)i * ldc + j;
    if constexpr (CDT == C_BF16) ((unsigned short*)c)[ci] = bf16_bits(sum);
    else ((float*)c)[ci] = sum;
}

A8W8_DEV float e2m1_to_f32(unsigned nibble)
{
    // +-{0, 0.5, 1, 1.5, 2, 3, 4, 6}: exponent field 0 is the subnormal pair {0, 0.5}
    const unsigned e = (nibble >> 1) & 3, m = nibble & 1;
    const float v = e == 0 ? 0.5f * (float)m : __builtin_ldexpf(1.0f + 0.5f * (float)m, (int)e - 1);
    return (nibble & 8) ? -v : v;
}

// MXFP4 x MXFP4 -> fp32 accumulate, any shape: packed E2M1 operands [rows][k/2] (even K in the low nibble),
// E8M0 scales row-major [rows][k/32] or tiled; the oracle's order of operations (product, times scale, add).
template <int CDT, bool TILED>
__global__ void __launch_bounds__(256) gemm_a4w4_general(const uint8_t* a, const uint8_t* b, const uint8_t* sfa, const uint8_t* sfb,
                                                         void* c, int m, int n, int k, int lda_bytes, int ldb_bytes, int ldc,
                                                         int stride_sfa, int stride_sfb, long long a_batch, long long b_batch,
                                                         long long c_batch, long long sfa_batch, long long sfb_batch)
{
#pragma clang fp contract(off)
    const int j = blockIdx.x * 16 + (threadIdx.x & 15);
    const int i = blockIdx.y * 16 + (threadIdx.x >> 4);
    const int batch = blockIdx.z;
    if (i >= m || j >= n) return;
    const uint8_t* ar = a + batch * a_batch + (long long)i * lda_bytes;
    const uint8_t* br = b + batch * b_batch + (long long)j * ldb_bytes;
    const uint8_t* ea = sfa + batch * sfa_batch;
    const uint8_t* eb = sfb + batch * sfb_batch;
    float sum = 0.f;
    for (int g = 0; g < k / 32; ++g) {
        const uint8_t xa = TILED ? ea[mx_tiled_index(m, i, g)] : ea[(long long)i * stride_sfa + g];
        const uint8_t xb = TILED ? eb[mx_tiled_index(n, j, g)] : eb[(long long)j * stride_sfb + g];
        const float scale = e8m0_pair_scale(xa, xb);
        for (int p = g * 32; p < g * 32 + 32; ++p) {
            const float av = e2m1_to_f32((ar[p >> 1] >> ((p & 1) * 4)) & 15u);
            const float bv = e2m1_to_f32((br[p >> 1] >> ((p & 1) * 4)) & 15u);
            const float prod = av * bv;
            const float term = prod * scale;
            sum = sum + term;
        }
    }
    const long long ci = batch * c_batch + (long long)i * ldc + j;
    if constexpr (CDT == C_BF16) ((unsigned short*)c)[ci] = bf16_bits(sum);
    else ((float*)c)[ci] = sum;
}

}  // namespace a8w8
