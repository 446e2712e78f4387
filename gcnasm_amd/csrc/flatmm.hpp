// Skinny-M ("flat") A8W8 GEMM over pre-shuffled weights for gfx950.
//
// B arrives as Bshuf[n/16][k/64][4][16][16 B]: one 1 KiB block per (16 rows of B, 64 K),
// ordered so that a 64-lane load of 16 bytes per lane is one contiguous 1 KiB read and lane
// (kq = lane/16, r = lane%16) receives K bytes [16kq, 16kq+16) of row r -- half of a
// 16 x 16 x 128 MFMA operand.  Two consecutive K blocks make one MFMA; the activation
// fragment is gathered with the same K order, so no data ever moves through LDS.
//
// The kernel is bound by HBM: B is read exactly once with non-temporal 16-byte loads.
// A workgroup is 8 waves that split K eight ways for the same NT weight tiles (all waves
// stream B concurrently, the activation fragment of a K block is shared by the NT tiles); the partial 16 x 16 accumulators are reduced through LDS and
// the dequantisation scales are applied in fp32 before the bf16 store.
#pragma once
#include "a8w8_device.hpp"

namespace a8w8 {

constexpr int FLAT_WAVES = 8;
constexpr int FLAT_THREADS = FLAT_WAVES * 64;

// Workgroup id -> (group of NT weight tiles, group of 16 activation rows).  The workgroups that stream the same weight
// tiles for different row groups get ids 8 apart and next to each other in that stride: the hardware deals consecutive
// ids to the 8 XCDs in turn, so they run on one XCD at the same time and all but the first find the weights in its L2.
A8W8_DEV void flat_work_of_block(int bid, int n_groups, int m_tiles, int& n_group, int& m_tile)
{
    if ((n_groups & 7) == 0) {
        const int rest = bid >> 3;
        m_tile = rest % m_tiles;
        n_group = (rest / m_tiles) * 8 + (bid & 7);
    } else {
        m_tile = bid % m_tiles;
        n_group = bid / m_tiles;
    }
}

template <int NT, int CDT, int MODE>
__global__ void __launch_bounds__(FLAT_THREADS) flatmm_a8w8(GemmParams p)
{
    static_assert(NT <= FLAT_WAVES, "wave t finishes weight tile t");
    __shared__ v4f red[FLAT_WAVES][NT][64];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = wave_uniform(tid >> 6);
    const int batch = blockIdx.z;
    const int r16 = lane & 15, kq = lane >> 4;

    const int n_tiles = p.n >> 4;
    const int k_tiles = p.k >> 6;
    int n_group, m_tile_;
    flat_work_of_block(blockIdx.x, (n_tiles + NT - 1) / NT, (p.m + 15) >> 4, n_group, m_tile_);
    const int nt0 = n_group * NT;
    const int m0 = m_tile_ * 16;

    // Wave t < NT writes tile t at the end: its lane holds C[m = r16][n = tile*16 + 4*kq .. +3].
    // Its scales are fetched now, so that the tail of the kernel is only reduce + store.
    const int cm = m0 + r16;
    const int cn = (nt0 + wave) * 16 + 4 * kq;
    const bool finisher = wave < NT && cm < p.m && nt0 + wave < n_tiles;
    float sa = 1.f;
    v4f sb = v4f{1.f, 1.f, 1.f, 1.f};
    if (finisher) {
        const float* sfa = (const float*)p.sfa + (long long)batch * p.sfa_batch;
        const float* sfb = (const float*)p.sfb + (long long)batch * p.sfb_batch;
        if constexpr (MODE == MODE_BF16 || MODE == MODE_MXT || MODE == MODE_BLOCK) {
            // bf16 operands carry no scales; MX scales go into the MFMAs, block scales into the K loop
        } else if constexpr (MODE == MODE_TENSOR) {
            sa = sfa[0] * sfb[0];
        } else {
            sa = sfa[cm];
            sb = v4f{sfb[cn], sfb[cn + 1], sfb[cn + 2], sfb[cn + 3]};
        }
    }

    const uint8_t* a_row = p.a + (long long)batch * p.a_batch + (long long)min(m0 + r16, p.m - 1) * p.lda + kq * 16;
    const uint8_t* b_base = p.b + (long long)batch * p.b_batch + lane * 16;
    const uint8_t* b_tile[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) b_tile[t] = b_base + (long long)min(nt0 + t, n_tiles - 1) * k_tiles * 1024;
    // MX scales in the tiled layout of the dense kernels (mx_tiled_index): a pair of K blocks is one 128-wide K
    // step ks; lane (r16, kq) scales 32-block kq of its row, whose byte for step ks sits at
    // ((ks / 4 * nblk + blk) * 2 + (ks / 2) % 2) * 512 + ((4x + y) * 4 + kq) * 8 + jp * 4 + par * 2 + ks % 2
    // with, for row 16 i + r16 of a 64-row block, x = (2 i + r16 / 8) % 4, y = r16 % 4, jp = i / 2, par = (r16 / 4) % 2
    const uint8_t* mx_a = nullptr;
    const uint8_t* mx_b[NT];
    int mx_nblk_a = 1, mx_nblk_b = 1;
    if constexpr (MODE == MODE_MXT) {
        auto lane_off = [&](int i) { return ((4 * ((2 * i + (r16 >> 3)) & 3) + (r16 & 3)) * 4 + kq) * 8 + (i >> 1) * 4 + ((r16 >> 2) & 1) * 2; };
        const int m_tile = m_tile_;
        mx_nblk_a = (p.m + 63) >> 6;
        mx_nblk_b = (p.n + 63) >> 6;
        mx_a = (const uint8_t*)p.sfa + (long long)batch * p.sfa_batch + (size_t)(m_tile >> 2) * 1024 + lane_off(m_tile & 3);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int nt = min(nt0 + t, n_tiles - 1);
            mx_b[t] = (const uint8_t*)p.sfb + (long long)batch * p.sfb_batch + (size_t)(nt >> 2) * 1024 + lane_off(nt & 3);
        }
    }

    // block scales (1x128 for A, 128x128 for B; the reference's layout): a pair of K blocks is one 128-wide scale
    // group, lane (r16, .) needs sfa[group][row m0 + r16] and, per weight tile, sfb[tile's 128-row block][group]
    const float* blk_a = nullptr;
    const float* blk_b[NT];
    if constexpr (MODE == MODE_BLOCK) {
        blk_a = (const float*)p.sfa + (long long)batch * p.sfa_batch + min(m0 + r16, p.m - 1);
#pragma unroll
        for (int t = 0; t < NT; ++t)
            blk_b[t] = (const float*)p.sfb + (long long)batch * p.sfb_batch + (long long)(min(nt0 + t, n_tiles - 1) >> 3) * p.stride_sfb;
    }

    // K blocks are consumed in pairs; this wave's share of the pairs
    const int pairs = (k_tiles + 1) >> 1;
    const int pp_begin = wave * pairs / FLAT_WAVES;
    const int pp_end = (wave + 1) * pairs / FLAT_WAVES;

    v4f acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = v4f{0.f, 0.f, 0.f, 0.f};

    struct Frag {
        v4i a[2];
        v4i b[NT][2];
        int sa, sb[NT];         // MX: the step's E8M0 byte of this lane's row and 32-block
        float fs[NT];           // block scales: sfa * sfb of the pair's scale group
    };
    auto load = [&](int pp, Frag& f) {
        const int kt0 = 2 * pp, kt1 = 2 * pp + 1;
        const bool has1 = kt1 < k_tiles;
        f.a[0] = *(const v4i*)(a_row + kt0 * 64);
        f.a[1] = has1 ? *(const v4i*)(a_row + kt1 * 64) : v4i{0, 0, 0, 0};
        size_t unit_a = 0, unit_b = 0;
        if constexpr (MODE == MODE_MXT) {
            unit_a = ((size_t)(pp >> 2) * mx_nblk_a * 2 + ((pp >> 1) & 1)) * 512 + (pp & 1);
            unit_b = ((size_t)(pp >> 2) * mx_nblk_b * 2 + ((pp >> 1) & 1)) * 512 + (pp & 1);
            f.sa = mx_a[unit_a];
        }
        float blk_sa = 1.f;
        if constexpr (MODE == MODE_BLOCK) blk_sa = blk_a[(long long)pp * p.stride_sfa];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            f.b[t][0] = __builtin_nontemporal_load((const v4i*)(b_tile[t] + (long long)kt0 * 1024));
            f.b[t][1] = has1 ? __builtin_nontemporal_load((const v4i*)(b_tile[t] + (long long)kt1 * 1024))
                             : v4i{0, 0, 0, 0};
            if constexpr (MODE == MODE_MXT) f.sb[t] = mx_b[t][unit_b];
            if constexpr (MODE == MODE_BLOCK) f.fs[t] = blk_sa * blk_b[t][pp];
        }
    };
    auto mma = [&](const Frag& f) {
        const v8i fa = v8i{f.a[0].x, f.a[0].y, f.a[0].z, f.a[0].w, f.a[1].x, f.a[1].y, f.a[1].z, f.a[1].w};
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const v8i fb = v8i{f.b[t][0].x, f.b[t][0].y, f.b[t][0].z, f.b[t][0].w,
                               f.b[t][1].x, f.b[t][1].y, f.b[t][1].z, f.b[t][1].w};
            if constexpr (MODE == MODE_BF16) {
                // bf16 weights: a 1 KiB block is 16 rows x 32 bf16, one 16x16x32 MFMA operand
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, f.b[t][0]),
                                                                 __builtin_bit_cast(v8bf, f.a[0]), acc[t], 0, 0, 0);
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, f.b[t][1]),
                                                                 __builtin_bit_cast(v8bf, f.a[1]), acc[t], 0, 0, 0);
            } else if constexpr (MODE == MODE_BLOCK) {
                // each 128-wide K group yields a partial tile that is rescaled into the running sum
                const v4f part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb, fa, v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                acc[t] += part * f.fs[t];
            } else if constexpr (MODE == MODE_MXT) {
                acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb, fa, acc[t], 0, 0, 0, f.sb[t], 0, f.sa);
            } else {
                acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb, fa, acc[t], 0, 0, 0, 0, 0, 0);
            }
        }
    };

    if (pp_begin < pp_end) {
        Frag f0, f1;
        load(pp_begin, f0);
        int pp = pp_begin;
        // two register stages, loads of the next pair in flight while the current one is used
        while (true) {
            if (pp + 1 < pp_end) load(pp + 1, f1);
            mma(f0);
            if (++pp >= pp_end) break;
            if (pp + 1 < pp_end) load(pp + 1, f0);
            mma(f1);
            if (++pp >= pp_end) break;
        }
    }

#pragma unroll
    for (int t = 0; t < NT; ++t) red[wave][t][lane] = acc[t];
    __syncthreads();

    if (finisher) {
        v4f s = red[0][wave][lane];
#pragma unroll
        for (int w = 1; w < FLAT_WAVES; ++w) s += red[w][wave][lane];
        s *= sb * sa;
        const long long ci = (long long)batch * p.c_batch + (long long)cm * p.ldc + cn;
        if constexpr (CDT == C_BF16) {
            unsigned short* dst = (unsigned short*)p.c + ci;
            if ((p.ldc & 3) == 0 && (((uintptr_t)p.c + 2 * (long long)batch * p.c_batch) & 7) == 0) {
                *(v4u16*)dst = v4u16{bf16_bits(s.x), bf16_bits(s.y), bf16_bits(s.z), bf16_bits(s.w)};
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) dst[e] = bf16_bits(s[e]);
            }
        } else {
            float* dst = (float*)p.c + ci;
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[e] = s[e];
        }
    }
}

// The MXFP4 flat GEMM: A and B hold packed E2M1 (two elements per byte), B pre-shuffled as the byte matrix
// [n][k/2] with the same 1 KiB blocks -- a block is 16 rows x 64 bytes = 16 rows x 128 elements, exactly one
// operand of the FP4 form of the 16 x 16 x 128 MFMA (lane (kq, r) supplies elements [32 kq, 32 kq + 32) of
// row r, one 32-element scale block).  E8M0 scales of both operands come in the tiled layout of the dense
// kernels (mx_tiled_index): the two bytes of (row, 32-block g) for the two 128-element blocks of a pair sit side
// by side, so a lane fetches one 16-bit word per tile and pair of blocks and op_sel picks the block's byte.
// p.k, p.lda count bytes (k/2 of the element counts); p.m, p.n count rows.
template <int NT, int CDT>
__global__ void __launch_bounds__(FLAT_THREADS) flatmm_a4w4(GemmParams p)
{
    static_assert(NT <= FLAT_WAVES, "wave t finishes weight tile t");
    __shared__ v4f red[FLAT_WAVES][NT][64];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = wave_uniform(tid >> 6);
    const int batch = blockIdx.z;
    const int r16 = lane & 15, kq = lane >> 4;

    const int n_tiles = p.n >> 4;
    const int k_tiles = p.k >> 6;                  // blocks of 64 bytes = 128 elements = one MFMA
    int n_group, m_tile;
    flat_work_of_block(blockIdx.x, (n_tiles + NT - 1) / NT, (p.m + 15) >> 4, n_group, m_tile);
    const int nt0 = n_group * NT;
    const int m0 = m_tile * 16;
    const int cm = m0 + r16;
    const int cn = (nt0 + wave) * 16 + 4 * kq;
    const bool finisher = wave < NT && cm < p.m && nt0 + wave < n_tiles;

    const uint8_t* a_row = p.a + (long long)batch * p.a_batch + (long long)min(m0 + r16, p.m - 1) * p.lda + kq * 16;
    const uint8_t* b_base = p.b + (long long)batch * p.b_batch + lane * 16;
    const uint8_t* b_tile[NT];
    // scale words: inside a 64-row block, row 16 i + r16 of 32-block kq lives at ((4x + y) * 4 + kq) * 8 + jp * 4 +
    // par * 2 + s with x = (2 i + r16 / 8) % 4, y = r16 % 4, jp = i / 2, par = (r16 / 4) % 2; the unit of (K group of
    // 512 elements, row block, pair of 128-element blocks) starts at ((kgroup * nblk + blk) * 2 + pair) * 512
    const int y = r16 & 3, par = (r16 >> 2) & 1;
    auto scale_lane_off = [&](int i) { return ((4 * ((2 * i + (r16 >> 3)) & 3) + y) * 4 + kq) * 8 + (i >> 1) * 4 + par * 2; };
    const int nblk_a = (p.m + 63) >> 6, nblk_b = (p.n + 63) >> 6;
    const uint8_t* sfa = (const uint8_t*)p.sfa + (long long)batch * p.sfa_batch + (size_t)(m_tile >> 2) * 1024 + scale_lane_off(m_tile & 3);
    const uint8_t* sfb[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int nt = min(nt0 + t, n_tiles - 1);
        b_tile[t] = b_base + (long long)nt * k_tiles * 1024;
        sfb[t] = (const uint8_t*)p.sfb + (long long)batch * p.sfb_batch + (size_t)(nt >> 2) * 1024 + scale_lane_off(nt & 3);
    }

    // pairs of blocks; this wave's share
    const int pairs = (k_tiles + 1) >> 1;
    const int pp_begin = wave * pairs / FLAT_WAVES;
    const int pp_end = (wave + 1) * pairs / FLAT_WAVES;

    v4f acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = v4f{0.f, 0.f, 0.f, 0.f};

    struct Frag {
        v4i a[2];
        v4i b[NT][2];
        int sa, sb[NT];
    };
    auto load = [&](int pp, Frag& f) {
        const int kt0 = 2 * pp, kt1 = 2 * pp + 1;
        const bool has1 = kt1 < k_tiles;
        f.a[0] = *(const v4i*)(a_row + kt0 * 64);
        f.a[1] = has1 ? *(const v4i*)(a_row + kt1 * 64) : v4i{0, 0, 0, 0};
        // pair pp of the tiled layout: K group pp / 2, pair pp % 2
        const size_t unit_a = ((size_t)(pp >> 1) * nblk_a * 2 + (pp & 1)) * 512, unit_b = ((size_t)(pp >> 1) * nblk_b * 2 + (pp & 1)) * 512;
        f.sa = *(const unsigned short*)(sfa + unit_a);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            f.b[t][0] = __builtin_nontemporal_load((const v4i*)(b_tile[t] + (long long)kt0 * 1024));
            f.b[t][1] = has1 ? __builtin_nontemporal_load((const v4i*)(b_tile[t] + (long long)kt1 * 1024))
                             : v4i{0, 0, 0, 0};
            f.sb[t] = *(const unsigned short*)(sfb[t] + unit_b);
        }
    };
    auto mma = [&](const Frag& f) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                (v8i{f.b[t][0].x, f.b[t][0].y, f.b[t][0].z, f.b[t][0].w, 0, 0, 0, 0}), (v8i{f.a[0].x, f.a[0].y, f.a[0].z, f.a[0].w, 0, 0, 0, 0}),
                acc[t], 4, 4, 0, f.sb[t], 0, f.sa);
            acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                (v8i{f.b[t][1].x, f.b[t][1].y, f.b[t][1].z, f.b[t][1].w, 0, 0, 0, 0}), (v8i{f.a[1].x, f.a[1].y, f.a[1].z, f.a[1].w, 0, 0, 0, 0}),
                acc[t], 4, 4, 1, f.sb[t], 1, f.sa);
        }
    };

    if (pp_begin < pp_end) {
        Frag f0, f1;
        load(pp_begin, f0);
        int pp = pp_begin;
        while (true) {
            if (pp + 1 < pp_end) load(pp + 1, f1);
            mma(f0);
            if (++pp >= pp_end) break;
            if (pp + 1 < pp_end) load(pp + 1, f0);
            mma(f1);
            if (++pp >= pp_end) break;
        }
    }

#pragma unroll
    for (int t = 0; t < NT; ++t) red[wave][t][lane] = acc[t];
    __syncthreads();

    if (finisher) {
        v4f s = red[0][wave][lane];
#pragma unroll
        for (int w = 1; w < FLAT_WAVES; ++w) s += red[w][wave][lane];
        const long long ci = (long long)batch * p.c_batch + (long long)cm * p.ldc + cn;
        if constexpr (CDT == C_BF16) {
            unsigned short* dst = (unsigned short*)p.c + ci;
            if ((p.ldc & 3) == 0 && (((uintptr_t)p.c + 2 * (long long)batch * p.c_batch) & 7) == 0) {
                *(v4u16*)dst = v4u16{bf16_bits(s.x), bf16_bits(s.y), bf16_bits(s.z), bf16_bits(s.w)};
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) dst[e] = bf16_bits(s[e]);
            }
        } else {
            float* dst = (float*)p.c + ci;
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[e] = s[e];
        }
    }
}

}  // namespace a8w8
