// fp8 <-> fp32 conversion helpers, weight pre-shuffle and the quantisation front end (gfx950).
#pragma once
#include "a8w8_device.hpp"

namespace a8w8 {

// ---------------------------------------------------------------- software E4M3 FNUZ
// The gfx942 dialect (bias 8, max 240, 0x80 = NaN, no -0) is not what gfx950 hardware
// converts to, so it is computed with integer arithmetic on the fp32 bit pattern.
A8W8_DEV uint8_t f32_to_e4m3_fnuz_sw(float x)
{
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const uint32_t sign = (u >> 31) << 7;
    const uint32_t au = u & 0x7fffffffu;
    if (au >= 0x7f800000u) return 0x80;                 // NaN and Inf have one code
    if (au > 0x43700000u) return (uint8_t)(sign | 0x7f); // beyond 240: largest finite
    const int e8 = (int)(au >> 23) - 127 + 8;           // exponent field in the fp8 format
    uint32_t mant = au & 0x7fffffu;
    uint32_t code, rem, half;
    if (e8 >= 1) {
        code = ((uint32_t)e8 << 3) | (mant >> 20);
        rem = mant & 0xfffffu;
        half = 0x80000u;
    } else {
        const int sh = 21 - e8;                          // 20 dropped bits + (1 - e8)
        if (sh > 25) return 0;                           // below half of the smallest subnormal
        mant |= 0x800000u;
        code = mant >> sh;
        rem = mant & ((1u << sh) - 1u);
        half = 1u << (sh - 1);
    }
    if (rem > half || (rem == half && (code & 1u))) ++code;   // nearest, ties to even
    if (code > 0x7fu) code = 0x7fu;
    if (code == 0) return 0;
    return (uint8_t)(sign | code);
}

A8W8_DEV float e4m3_fnuz_to_f32_sw(uint8_t c)
{
    if (c == 0) return 0.f;
    if (c == 0x80) return __builtin_bit_cast(float, 0x7F800001u);
    uint32_t sign = (uint32_t)(c >> 7) << 31;
    int e = (c >> 3) & 15;
    uint32_t m = c & 7;
    if (e == 0) {                       // subnormal: shift the leading one into place
        const int lz = __builtin_clz(m) - 29;   // 0 for m>=4, 1 for m>=2, 2 for m==1
        m = (m << (lz + 1)) & 7;
        e = -lz;
    }
    return __builtin_bit_cast(float, sign | ((uint32_t)(e + 127 - 8) << 23) | (m << 20));
}

// to_fp8_raw_from_fp32 of the reference (cvt_fp8/test.cpp:21-43) on this hardware.
A8W8_DEV float clamp240_unless_special(float v)
{
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    if ((u & 0x7F800000u) != 0x7F800000u) v = __builtin_amdgcn_fmed3f(v, 240.0f, -240.0f);
    return v;
}

// One thread converts four consecutive floats into one packed word:
// two packed hardware converts into the low halves, merged by a byte permute
// (the sequence of pk_cvt_fp8x4_fp32x4_rne, pk_cvt/test.cpp:220-257).
template <int DIALECT, int CLAMP>
__global__ void __launch_bounds__(256) cvt_f32_to_e4m3_kernel(const float* src, uint8_t* dst, size_t n)
{
    const size_t q = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t i0 = q * 4;
    if (i0 >= n) return;
    float s[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        s[e] = i0 + e < n ? src[i0 + e] : 0.f;
        if (CLAMP) s[e] = clamp240_unless_special(s[e]);
    }
    uint32_t word;
    if (DIALECT == 0) {
        const uint32_t x = __builtin_amdgcn_cvt_pk_fp8_f32(s[0], s[1], 0, false);
        const uint32_t y = __builtin_amdgcn_cvt_pk_fp8_f32(s[2], s[3], 0, false);
        word = __builtin_amdgcn_perm(y, x, 0x05040100);
    } else {
        word = (uint32_t)f32_to_e4m3_fnuz_sw(s[0]) | ((uint32_t)f32_to_e4m3_fnuz_sw(s[1]) << 8) |
               ((uint32_t)f32_to_e4m3_fnuz_sw(s[2]) << 16) | ((uint32_t)f32_to_e4m3_fnuz_sw(s[3]) << 24);
    }
    if (i0 + 3 < n && ((uintptr_t)dst & 3) == 0) {
        *(uint32_t*)(dst + i0) = word;
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (i0 + e < n) dst[i0 + e] = (uint8_t)(word >> (8 * e));
    }
}

template <int DIALECT>
__global__ void __launch_bounds__(256) cvt_e4m3_to_f32_kernel(const uint8_t* src, float* dst, size_t n)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint8_t c = src[i];
    dst[i] = DIALECT == 0 ? __builtin_amdgcn_cvt_f32_fp8((int)c, 0) : e4m3_fnuz_to_f32_sw(c);
}

// Row-major B[n][k] -> Bshuf[n/16][k/64][4][16][16 B]; one thread moves 16 bytes.
__global__ void __launch_bounds__(256) preshuffle_b_kernel(const uint8_t* b, uint8_t* out, int n, int k)
{
    const long long o = (long long)blockIdx.x * 256 + threadIdx.x;   // 16-byte unit in the output
    const long long total = (long long)n * k / 16;
    if (o >= total) return;
    const int r = (int)(o & 15);
    const int kq = (int)((o >> 4) & 3);
    const long long blk = o >> 6;
    const int k_tiles = k >> 6;
    const int kt = (int)(blk % k_tiles);
    const int nt = (int)(blk / k_tiles);
    const uint8_t* src = b + (long long)(nt * 16 + r) * k + kt * 64 + kq * 16;
    v4i v;
    if (((uintptr_t)src & 15) == 0) v = *(const v4i*)src;
    else __builtin_memcpy(&v, src, 16);
    *(v4i*)(out + o * 16) = v;
}

// ------------------------------------------------------------ quantisation front end
A8W8_DEV float wave_max(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

A8W8_DEV uint8_t quant_one(float x, float scale)
{
    const float q = __fdiv_rn(x, scale);
    const uint32_t w = __builtin_amdgcn_cvt_pk_fp8_f32(q, q, 0, false);
    return (uint8_t)w;
}

// per-row scale = amax(row)/448; one workgroup per row
__global__ void __launch_bounds__(256) quant_rowwise_kernel(const float* src, int k, int ld, uint8_t* q, float* scale)
{
    __shared__ float part[4];
    const int row = blockIdx.x;
    const float* x = src + (long long)row * ld;
    float amax = 0.f;
    for (int i = threadIdx.x; i < k; i += 256) amax = fmaxf(amax, fabsf(x[i]));
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    const float s = amax > 0.f ? __fdiv_rn(amax, 448.0f) : 1.0f;   // an all-zero group keeps scale 1
    if (threadIdx.x == 0) scale[row] = s;
    for (int i = threadIdx.x; i < k; i += 256) q[(long long)row * k + i] = quant_one(x[i], s);
}

// per-tensor scale = amax(all)/448 in three steps over the caller's one-float scale slot: clear it, fold
// every workgroup's |x| maximum into it (non-negative floats order like their bit patterns), quantise with
// amax/448, and finally turn the slot from amax into the scale.
__global__ void quant_tensor_clear_kernel(float* scale) { *scale = 0.f; }
__global__ void __launch_bounds__(256) quant_tensor_amax_kernel(const float* src, int rows, int k, int ld, float* scale)
{
    __shared__ float part[4];
    const long long total = (long long)rows * k;
    float amax = 0.f;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256)
        amax = fmaxf(amax, fabsf(src[(i / k) * ld + i % k]));
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = amax;
    __syncthreads();
    if (threadIdx.x == 0) {
        amax = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
        atomicMax((unsigned int*)scale, __float_as_uint(amax));
    }
}
__global__ void __launch_bounds__(256) quant_tensor_apply_kernel(const float* src, int rows, int k, int ld, uint8_t* q,
                                                                 const float* amax_slot)
{
    const long long total = (long long)rows * k;
    const float amax = *amax_slot;
    const float s = amax > 0.f ? __fdiv_rn(amax, 448.0f) : 1.0f;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256)
        q[i] = quant_one(src[(i / k) * ld + i % k], s);
}
__global__ void quant_tensor_finish_kernel(float* scale)
{
    const float amax = *scale;
    *scale = amax > 0.f ? __fdiv_rn(amax, 448.0f) : 1.0f;
}

// 1 x 128 blocks: one wave per (row, 128-group); scale stored [k/128][rows]
__global__ void __launch_bounds__(256) quant_1x128_kernel(const float* src, int rows, int k, int ld, uint8_t* q,
                                                          float* scale)
{
    const int groups = k >> 7;
    const long long w = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (w >= (long long)rows * groups) return;
    const int row = (int)(w / groups), g = (int)(w % groups);
    const int lane = threadIdx.x & 63;
    const float* x = src + (long long)row * ld + g * 128;
    const float v0 = x[lane], v1 = x[lane + 64];
    const float amax = wave_max(fmaxf(fabsf(v0), fabsf(v1)));
    const float s = amax > 0.f ? __fdiv_rn(amax, 448.0f) : 1.0f;   // an all-zero group keeps scale 1
    if (lane == 0) scale[(long long)g * rows + row] = s;
    uint8_t* o = q + (long long)row * k + g * 128;
    o[lane] = quant_one(v0, s);
    o[lane + 64] = quant_one(v1, s);
}

// 128 x 128 blocks: one workgroup per block; scale stored [rows/128][k/128]
__global__ void __launch_bounds__(256) quant_128x128_kernel(const float* src, int k, int ld, uint8_t* q, float* scale)
{
    __shared__ float part[4];
    const int gk = blockIdx.x, gr = blockIdx.y;
    const float* x = src + (long long)gr * 128 * ld + gk * 128;
    float amax = 0.f;
    for (int i = threadIdx.x; i < 128 * 128; i += 256) amax = fmaxf(amax, fabsf(x[(long long)(i >> 7) * ld + (i & 127)]));
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    const float s = amax > 0.f ? __fdiv_rn(amax, 448.0f) : 1.0f;   // an all-zero group keeps scale 1
    if (threadIdx.x == 0) scale[(long long)gr * gridDim.x + gk] = s;
    uint8_t* o = q + (long long)gr * 128 * k + gk * 128;
    for (int i = threadIdx.x; i < 128 * 128; i += 256)
        o[(long long)(i >> 7) * k + (i & 127)] = quant_one(x[(long long)(i >> 7) * ld + (i & 127)], s);
}

// MX: one E8M0 exponent per 32 K-elements, e = ceil(log2(amax/448)) clamped to [-127, 127]
// computed exactly from the fp32 exponent/mantissa fields; 32 lanes per block.
template <bool TILED>
__global__ void __launch_bounds__(256) quant_mx_kernel(const float* src, int rows, int k, int ld, uint8_t* q,
                                                       uint8_t* scale)
{
    const int blocks = k >> 5;
    const long long idx = ((long long)blockIdx.x * 256 + threadIdx.x) >> 5;
    if (idx >= (long long)rows * blocks) return;
    const int row = (int)(idx / blocks), g = (int)(idx % blocks);
    const int l = threadIdx.x & 31;
    const float v = src[(long long)row * ld + g * 32 + l];
    float amax = fabsf(v);
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    const float t = __fdiv_rn(amax, 448.0f);
    int e = -127;
    if (t > 0.f) {
        int ex;
        const float f = frexpf(t, &ex);          // t = f * 2^ex, f in [0.5, 1)
        e = (f == 0.5f) ? ex - 1 : ex;
        e = max(-127, min(127, e));
    }
    if (l == 0) scale[TILED ? mx_tiled_index(rows, row, g) : (size_t)row * blocks + g] = (uint8_t)(e + 127);
    const float qv = ldexpf(v, -e);
    const uint32_t w = __builtin_amdgcn_cvt_pk_fp8_f32(qv, qv, 0, false);
    q[(long long)row * k + g * 32 + l] = (uint8_t)w;
}

// natural [rows][k/32] E8M0 scales (row stride `stride` bytes) -> the tiled layout of mx_tiled_index.
// One thread per output dword: two tiles x two K steps of one (64-row block, r16, g, jp).
// Consecutive threads write consecutive dwords.  Rows past `rows` and blocks past k get 127
// (scale 1.0; their products are never formed or never stored).
// MXFP4: one E8M0 exponent per 32 K-elements, e = ceil(log2(amax/6)) clamped to [-127, 127]; elements
// become E2M1 (round to nearest, ties to the even mantissa bit, saturating at 6), two per byte with
// the even K index in the low nibble.  32 lanes per block; even lanes write the byte.
A8W8_DEV unsigned e2m1_encode(float x)
{
    const float a = fabsf(x);
    const unsigned code = (a > 0.25f) + (a >= 0.75f) + (a > 1.25f) + (a >= 1.75f) + (a > 2.5f) + (a >= 3.5f) + (a > 5.0f);
    return ((__float_as_uint(x) >> 31) << 3) | (a != a ? 7u : code);
}
template <bool TILED>
__global__ void __launch_bounds__(256) quant_mxfp4_kernel(const float* src, int rows, int k, int ld, uint8_t* q,
                                                          uint8_t* scale)
{
    const int blocks = k >> 5;
    const long long idx = ((long long)blockIdx.x * 256 + threadIdx.x) >> 5;
    if (idx >= (long long)rows * blocks) return;
    const int row = (int)(idx / blocks), g = (int)(idx % blocks);
    const int l = threadIdx.x & 31;
    const float v = src[(long long)row * ld + g * 32 + l];
    float amax = fabsf(v);
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    const float t = __fdiv_rn(amax, 6.0f);
    int e = -127;
    if (t > 0.f) {
        int ex;
        const float f = frexpf(t, &ex);          // t = f * 2^ex, f in [0.5, 1)
        e = (f == 0.5f) ? ex - 1 : ex;
        e = max(-127, min(127, e));
    }
    if (l == 0) scale[TILED ? mx_tiled_index(rows, row, g) : (size_t)row * blocks + g] = (uint8_t)(e + 127);
    const unsigned code = e2m1_encode(ldexpf(v, -e));
    const unsigned hi = __shfl_down(code, 1, 64);
    if ((l & 1) == 0) q[(long long)row * (k >> 1) + ((g * 32 + l) >> 1)] = (uint8_t)(code | (hi << 4));
}

// ------------------------------------------------------------ vectorised quantisers
// The kernels above move one element per thread (4-byte loads, 1-byte stores).  When rows are
// 16-byte aligned (src, ld % 4 == 0, k % 4 == 0) the kernels below do the same arithmetic on four
// elements per thread per chunk: 16-byte loads, one packed store, same bits out.
A8W8_DEV uint32_t pack4_e4m3(float a, float b, float c, float d)
{
    uint32_t w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    return __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
}
A8W8_DEV int mx_block_exponent(float amax, float top)
{
    const float t = __fdiv_rn(amax, top);
    int e = -127;
    if (t > 0.f) {
        int ex;
        const float f = frexpf(t, &ex);          // t = f * 2^ex, f in [0.5, 1)
        e = (f == 0.5f) ? ex - 1 : ex;
        e = max(-127, min(127, e));
    }
    return e;
}

// 16 bytes of an input that is read once: a non-temporal load (the line is not kept in L2 in place of something that
// will be read again; 8192 x 8192 fp32 to FP8 with row scales 58.9 -> 54.2 us, to MXFP8 56.6 -> 54.1 us)
A8W8_DEV float4 load_once4(const float* p)
{
    const v4f t = __builtin_nontemporal_load((const v4f*)p);
    return make_float4(t.x, t.y, t.z, t.w);
}

// MX E4M3 with one E8M0 exponent per 32 elements.  A wave takes 1024 consecutive elements of the
// flattened [rows, k] array as four chunks of 256: lane l owns elements 4l..4l+3 of each chunk, eight
// lanes share a block.  Every load and store instruction of a wave covers one contiguous run of memory;
// all loads are issued before any chunk is processed.
constexpr int QUANT_MX_CHUNKS = 4;
template <bool TILED>
__global__ void __launch_bounds__(256) quant_mx_vec_kernel(const float* __restrict__ src, int rows, int k, int ld,
                                                           uint8_t* __restrict__ q, uint8_t* __restrict__ scale)
{
    const unsigned total = (unsigned)rows * (unsigned)k;            // < 2^31 (checked by the host)
    const unsigned wave = (blockIdx.x * 256u + threadIdx.x) >> 6;
    const unsigned lane = threadIdx.x & 63;
    const int blocks = k >> 5;
    constexpr int CH = QUANT_MX_CHUNKS;
    unsigned row[CH], col[CH];
    bool live[CH];
    float4 v[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const unsigned e0 = wave * (256u * CH) + c * 256u + lane * 4u;
        live[c] = e0 < total;
        row[c] = live[c] ? e0 / (unsigned)k : 0u;
        col[c] = live[c] ? e0 % (unsigned)k : 0u;
        v[c] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live[c]) v[c] = load_once4(src + (size_t)row[c] * ld + col[c]);
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        float amax = fmaxf(fmaxf(fabsf(v[c].x), fabsf(v[c].y)), fmaxf(fabsf(v[c].z), fabsf(v[c].w)));
#pragma unroll
        for (int off = 4; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
        const int e = mx_block_exponent(amax, 448.0f);
        if (!live[c]) continue;
        if ((lane & 7) == 0) {
            const int g = (int)(col[c] >> 5);
            scale[TILED ? mx_tiled_index(rows, (int)row[c], g) : (size_t)row[c] * blocks + g] = (uint8_t)(e + 127);
        }
        *(uint32_t*)(q + (size_t)row[c] * k + col[c]) =
            pack4_e4m3(ldexpf(v[c].x, -e), ldexpf(v[c].y, -e), ldexpf(v[c].z, -e), ldexpf(v[c].w, -e));
    }
}

// MXFP4 (packed E2M1): lane l owns eight consecutive elements (two 16-byte loads, one 4-byte store),
// four lanes share a block, a wave takes 512 consecutive elements.
template <bool TILED>
__global__ void __launch_bounds__(256) quant_mxfp4_vec_kernel(const float* __restrict__ src, int rows, int k, int ld,
                                                              uint8_t* __restrict__ q, uint8_t* __restrict__ scale)
{
    const unsigned total = (unsigned)rows * (unsigned)k;            // < 2^31 (checked by the host)
    const unsigned e0 = (blockIdx.x * 256u + threadIdx.x) * 8u;
    const bool live = e0 < total;
    const unsigned row = live ? e0 / (unsigned)k : 0u, col = live ? e0 % (unsigned)k : 0u;
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
    if (live) {
        const float4* p = (const float4*)(src + (size_t)row * ld + col);
        a = p[0];
        b = p[1];
    }
    float amax = fmaxf(fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w))),
                       fmaxf(fmaxf(fabsf(b.x), fabsf(b.y)), fmaxf(fabsf(b.z), fabsf(b.w))));
#pragma unroll
    for (int off = 2; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    const int e = mx_block_exponent(amax, 6.0f);
    if (!live) return;
    if ((threadIdx.x & 3) == 0) {
        const int g = (int)(col >> 5);
        scale[TILED ? mx_tiled_index(rows, (int)row, g) : (size_t)row * (k >> 5) + g] = (uint8_t)(e + 127);
    }
    const float x[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    unsigned w = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) w |= e2m1_encode(ldexpf(x[i], -e)) << (4 * i);     // even K in the low nibble
    *(uint32_t*)(q + (size_t)row * (k >> 1) + (col >> 1)) = w;
}

// per-row scale, one workgroup per row.  HOLD: the row has at most 8192 elements and stays in registers
// between the amax pass and the quantisation (one read of the input); otherwise it is read twice.
template <bool HOLD>
__global__ void __launch_bounds__(256) quant_rowwise_vec_kernel(const float* __restrict__ src, int k, int ld,
                                                                uint8_t* __restrict__ q, float* __restrict__ scale)
{
    __shared__ float part[4];
    const int row = blockIdx.x;
    const float* x = src + (size_t)row * ld;
    float4 held[8];
    float amax = 0.f;
    if constexpr (HOLD) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = threadIdx.x * 4 + u * 1024;
            held[u] = i < k ? load_once4(x + i) : make_float4(0.f, 0.f, 0.f, 0.f);
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(held[u].x), fabsf(held[u].y)), fmaxf(fabsf(held[u].z), fabsf(held[u].w))));
        }
    } else {
        for (int i = threadIdx.x * 4; i < k; i += 1024) {
            const float4 v = *(const float4*)(x + i);
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        }
    }
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    const float s = amax > 0.f ? __fdiv_rn(amax, 448.0f) : 1.0f;   // an all-zero group keeps scale 1
    if (threadIdx.x == 0) scale[row] = s;
    if constexpr (HOLD) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = threadIdx.x * 4 + u * 1024;
            if (i < k)
                *(uint32_t*)(q + (size_t)row * k + i) = pack4_e4m3(__fdiv_rn(held[u].x, s), __fdiv_rn(held[u].y, s),
                                                                   __fdiv_rn(held[u].z, s), __fdiv_rn(held[u].w, s));
        }
    } else {
        for (int i = threadIdx.x * 4; i < k; i += 1024) {
            const float4 v = *(const float4*)(x + i);
            *(uint32_t*)(q + (size_t)row * k + i) =
                pack4_e4m3(__fdiv_rn(v.x, s), __fdiv_rn(v.y, s), __fdiv_rn(v.z, s), __fdiv_rn(v.w, s));
        }
    }
}

// 1 x 128 blocks: 32 lanes per (row, 128-group); a half wave takes four consecutive groups, loads first.
// Scale stored [k/128][rows].
constexpr int QUANT_1X128_GROUPS = 4;
__global__ void __launch_bounds__(256) quant_1x128_vec_kernel(const float* __restrict__ src, int rows, int k, int ld,
                                                              uint8_t* __restrict__ q, float* __restrict__ scale)
{
    constexpr int G = QUANT_1X128_GROUPS;
    const int groups = k >> 7;
    const long long total = (long long)rows * groups;
    const long long w0 = (((long long)blockIdx.x * 256 + threadIdx.x) >> 5) * G;
    const int l = threadIdx.x & 31;
    float4 v[G];
    int row[G], g[G];
    bool live[G];
#pragma unroll
    for (int u = 0; u < G; ++u) {
        live[u] = w0 + u < total;
        row[u] = live[u] ? (int)((w0 + u) / groups) : 0;
        g[u] = live[u] ? (int)((w0 + u) % groups) : 0;
        v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live[u]) v[u] = load_once4(src + (size_t)row[u] * ld + g[u] * 128 + 4 * l);
    }
#pragma unroll
    for (int u = 0; u < G; ++u) {
        float amax = fmaxf(fmaxf(fabsf(v[u].x), fabsf(v[u].y)), fmaxf(fabsf(v[u].z), fabsf(v[u].w)));
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
        if (!live[u]) continue;
        const float s = amax > 0.f ? __fdiv_rn(amax, 448.0f) : 1.0f;   // an all-zero group keeps scale 1
        if (l == 0) scale[(size_t)g[u] * rows + row[u]] = s;
        *(uint32_t*)(q + (size_t)row[u] * k + g[u] * 128 + 4 * l) =
            pack4_e4m3(__fdiv_rn(v[u].x, s), __fdiv_rn(v[u].y, s), __fdiv_rn(v[u].z, s), __fdiv_rn(v[u].w, s));
    }
}

// per-tensor scale over a contiguous array (ld == k): the amax and apply passes on 16-byte units, four
// units per thread and iteration (loads first)
__global__ void __launch_bounds__(256) quant_tensor_amax_vec_kernel(const float4* __restrict__ src, size_t units, float* scale)
{
    __shared__ float part[4];
    float amax = 0.f;
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < units; i += 4 * stride) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = i + u * stride < units ? src[i + u * stride] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int u = 0; u < 4; ++u)
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[u].x), fabsf(v[u].y)), fmaxf(fabsf(v[u].z), fabsf(v[u].w))));
    }
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = amax;
    __syncthreads();
    if (threadIdx.x == 0) {
        amax = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
        // thousands of atomics on one address take longer than the pass over the data: only a
        // workgroup that would raise the maximum sends one
        if (__float_as_uint(amax) > __hip_atomic_load((unsigned int*)scale, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
            atomicMax((unsigned int*)scale, __float_as_uint(amax));
    }
}
__global__ void __launch_bounds__(256) quant_tensor_apply_vec_kernel(const float4* __restrict__ src, size_t units,
                                                                     uint32_t* __restrict__ q, const float* __restrict__ amax_slot)
{
    const float amax = *amax_slot;
    const float s = amax > 0.f ? __fdiv_rn(amax, 448.0f) : 1.0f;
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < units; i += 4 * stride) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = i + u * stride < units ? src[i + u * stride] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (i + u * stride < units)
                q[i + u * stride] = pack4_e4m3(__fdiv_rn(v[u].x, s), __fdiv_rn(v[u].y, s), __fdiv_rn(v[u].z, s), __fdiv_rn(v[u].w, s));
    }
}

// One launch for one or two scale arrays (the A-side and the B-side scales of a GEMM).  A group of
// 64 threads handles one 1 KiB unit (64 rows x 16 K blocks): thread r copies the 16 bytes of row r
// into LDS, then thread t gathers and writes bytes 16t..16t+15 of the unit.  256 threads = 4 units.
__global__ void __launch_bounds__(256) mx_tile_scales_kernel(const uint8_t* sf0, int rows0, int stride0, uint8_t* out0,
                                                             const uint8_t* sf1, int rows1, int stride1, uint8_t* out1,
                                                             int k)
{
    __shared__ uint8_t lds[4][64 * 16];
    const int t = threadIdx.x & 63, sub = threadIdx.x >> 6;
    size_t unit = (size_t)blockIdx.x * 4 + sub;
    const size_t units0 = mx_tiled_bytes(rows0, k) >> 10;
    const uint8_t* sf = sf0;
    uint8_t* out = out0;
    int rows = rows0, stride = stride0;
    bool live = true;
    if (unit >= units0) {
        unit -= units0;
        sf = sf1;
        out = out1;
        rows = rows1;
        stride = stride1;
        live = sf1 != nullptr && unit < (mx_tiled_bytes(rows1, k) >> 10);
    }
    const int blocks = k >> 5;
    if (live) {
        // the workgroup's four units are consecutive K groups of one 64-row block: together they read 64
        // contiguous bytes of every row (the units themselves lie K group by K group in the output)
        const int nblk = (rows + 63) >> 6, kgroups = (k + 511) >> 9;
        const int kg = (int)(unit % kgroups), blk = (int)(unit / kgroups);
        unit = (size_t)kg * nblk + blk;
        const int row = blk * 64 + t;
        const uint8_t* src = sf + (size_t)row * stride + kg * 16;
        const bool vec = row < rows && kg * 16 + 16 <= blocks && (((uintptr_t)src) & 3) == 0;
        uint32_t w[4] = {0x7f7f7f7fu, 0x7f7f7f7fu, 0x7f7f7f7fu, 0x7f7f7f7fu};
        if (vec) {
#pragma unroll
            for (int q = 0; q < 4; ++q) w[q] = ((const uint32_t*)src)[q];
        } else if (row < rows) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t v = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) v |= (uint32_t)(kg * 16 + 4 * q + e < blocks ? src[4 * q + e] : 127u) << (8 * e);
                w[q] = v;
            }
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) ((uint32_t*)lds[sub])[t * 4 + q] = w[q];
    }
    __syncthreads();
    if (live) {
        const int pair = t >> 5, r16 = (t >> 1) & 15;
        uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int st = e & 1, par = (e >> 1) & 1, jp = (e >> 2) & 1, g = (t & 1) * 2 + (e >> 3);
            const int row = 32 * jp + 8 * (r16 >> 2) + 4 * par + (r16 & 3);
            w[e >> 2] |= (uint32_t)lds[sub][row * 16 + pair * 8 + st * 4 + g] << (8 * (e & 3));
        }
        *(v4i*)(out + (unit << 10) + t * 16) = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
    }
}

// 127 everywhere (tiled layout), for producers that then write only the real (row, block) positions.
__global__ void __launch_bounds__(256) mx_tiled_fill_kernel(uint32_t* scale, size_t dwords)
{
    const size_t d = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (d < dwords) scale[d] = 0x7f7f7f7fu;
}

}  // namespace a8w8
