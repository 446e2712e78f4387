// Dense A8W8 GEMM for gfx950: 256 x 256 x 128 tile, 8 waves (4 along M x 2 along N),
// each wave owning a 64 x 128 block of C as 4 x 8 MFMA tiles of 16 x 16 x 128.
//
// Data path: A and B tiles go global -> LDS with 16-byte direct-to-LDS buffer loads, two
// LDS stages (2 x 64 KiB), one barrier per K step.  LDS rows are 128 bytes (one K step of
// one matrix row); the 16-byte slots of a row are XOR-swizzled with (row & 7) on the
// global-address side (the direct-to-LDS write itself is always wave-linear) and
// un-swizzled by the readers, which keeps the 64-lane ds_read_b128 free of bank conflicts.
//
// MFMA operand roles are swapped with respect to the matrix names: rows of B (index n)
// feed the MFMA "A" operand and rows of A (index m) the "B" operand, so that a lane ends
// up holding C[m = lane%16][n = 4*(lane/16) .. +3]: four consecutive n, one 8-byte store
// of bf16, and one A-side scale per lane per tile.
#pragma once
#include "a8w8_device.hpp"

namespace a8w8 {

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int GEMM_THREADS = 512;
constexpr int STAGE_BYTES = (BM + BN) * BK;          // 65536
constexpr int GEMM_LDS_BYTES = 2 * STAGE_BYTES;      // 131072
// MX only: E8M0 scales of 4 K steps (16 bytes per row, 256 A rows then 256 B rows), two buffers
constexpr int MX_GROUP_BYTES = (BM + BN) * 16;       // 8192
constexpr int GEMM_LDS_BYTES_MX = GEMM_LDS_BYTES + 2 * MX_GROUP_BYTES;
constexpr int WAVE_M = 64, WAVE_N = 128;
constexpr int TM = WAVE_M / 16, TN = WAVE_N / 16;    // 4 x 8 MFMA tiles per wave

// Workgroup id -> tile.  Consecutive workgroup ids land on different XCDs (round-robin over
// 8), each with its own L2, so ids are first regrouped so that one XCD works on a
// contiguous run of tiles; inside the run, tiles are walked down 8 tile-rows before moving
// to the next tile-column so that concurrently resident tiles share A rows and B rows.
A8W8_DEV void tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn)
{
    const int nt = tiles_m * tiles_n;
    int id = bid;
    if ((nt & 7) == 0) id = (bid & 7) * (nt >> 3) + (bid >> 3);
    constexpr int GROUP = 8;
    const int per_group = GROUP * tiles_n;
    const int group = id / per_group;
    const int first_m = group * GROUP;
    const int gsz = min(tiles_m - first_m, GROUP);
    const int in_group = id - group * per_group;
    tm = first_m + in_group % gsz;
    tn = in_group / gsz;
}

template <int MODE, int CDT>
__global__ void __launch_bounds__(GEMM_THREADS, 1) gemm_a8w8_tile256(GemmParams p)
{
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = wave_uniform(tid >> 6);
    const int wave_m = wave >> 1, wave_n = wave & 1;
    const int batch = blockIdx.z;

    int tile_m, tile_n;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const uint8_t* a_base = p.a + (long long)batch * p.a_batch;
    const uint8_t* b_base = p.b + (long long)batch * p.b_batch;
    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(a_base, (uint32_t)(p.m - 1) * p.lda + p.k);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(b_base, b_extent_bytes(p));

    // ---- global -> LDS assignment.  A stage holds 32 A chunks then 32 B chunks of 1 KiB
    // (8 rows x 128 B).  Wave w fills chunks w, w+8, w+16, w+24 of each matrix; lane i of
    // the load lands at chunk*1024 + 16*i = row (i/8), slot (i%8), and therefore fetches
    // K-piece slot ^ key(row), key(row) = row & 7 = i/8.
    const int ld_row = wave * 8 + (lane >> 3);
    const int ld_piece = (lane & 7) ^ (lane >> 3);
    int voff_a[4], voff_b[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        voff_a[j] = min(m0 + ld_row + 64 * j, p.m - 1) * p.lda + ld_piece * 16;
        voff_b[j] = b_lane_offset(p, min(n0 + ld_row + 64 * j, p.n - 1), ld_piece * 16);
    }
    auto issue_stage = [&](int stage, int kstep) {
        A8W8_LDS char* s = (A8W8_LDS char*)smem + stage * STAGE_BYTES + wave * 1024;
        const int koff = kstep * BK;
#pragma unroll
        for (int j = 0; j < 4; ++j) load_to_lds_16(rsrc_a, s + j * 8192, voff_a[j], koff);
#pragma unroll
        for (int j = 0; j < 4; ++j) load_to_lds_16(rsrc_b, s + BM * BK + j * 8192, voff_b[j], kstep << p.b_kshift);
    };

    // ---- LDS -> register addresses.  The 16 x 16 x 128 FP8 MFMA takes, from lane
    // (r = lane%16, g = lane/16), K bytes [16g, 16g+16) in its first four operand registers
    // and [64+16g, 64+16g+16) in the last four (measured with the block-scaled form, whose
    // scale of lane (r, g) covers K [32g, 32g+32)).  So a lane reads K-pieces g and g+4 of
    // tile row r; un-swizzled slot = piece ^ (row & 7), and row & 7 = lane & 7 for every tile.
    const int r16 = lane & 15, g = lane >> 4;
    int rd_a[2], rd_b[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int slot = (g + 4 * h) ^ (lane & 7);
        rd_a[h] = (wave_m * WAVE_M + r16) * BK + (slot << 4);
        rd_b[h] = BM * BK + (wave_n * WAVE_N + r16) * BK + (slot << 4);
    }
    auto read_frag = [&](int stage, const int (&base)[2], int t) -> v8i {
        const char* s = smem + stage * STAGE_BYTES + t * (16 * BK);
        const v4i lo = *(const v4i*)(s + base[0]);
        const v4i hi = *(const v4i*)(s + base[1]);
        return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    };

    // rows / columns this lane owns in C, and the rows whose scales it needs
    const int cm_base = m0 + wave_m * WAVE_M + r16;          // + 16*tm
    const int cn_base = n0 + wave_n * WAVE_N + 4 * g;        // + 16*tn + i

    v4f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    const int nk = p.k / BK;

    // ---- per-K-step scales (BLOCK: fp32, MX: E8M0 bytes), fetched one step ahead
    const float* sfa_f = (const float*)p.sfa + (long long)batch * p.sfa_batch;
    const float* sfb_f = (const float*)p.sfb + (long long)batch * p.sfb_batch;
    const uint8_t* sfa_e = (const uint8_t*)p.sfa + (long long)batch * p.sfa_batch;
    const uint8_t* sfb_e = (const uint8_t*)p.sfb + (long long)batch * p.sfb_batch;
    float blk_sa[TM], blk_sa_next[TM];
    float blk_sb_next = 0.f;
    int mx_sa[TM], mx_sb[TN], mx_sa_next[TM], mx_sb_next[TN];
    // MX: thread t stages the 16 scale bytes (4 K steps) of A row m0+t (t < 256) or B row
    // n0+t-256 with one direct-to-LDS load per group of 4 K steps; lanes then pick single
    // bytes with ds_read_u8, one K step ahead of their use.
    __amdgpu_buffer_rsrc_t rsrc_sf = rsrc_a;
    int voff_sf = 0, rd_sfa = 0, rd_sfb = 0;
    if constexpr (MODE == MODE_MX) {
        const bool is_b = wave >= 4;                      // wave-uniform: waves 0-3 stage A rows, 4-7 B rows
        const int rows = is_b ? p.n : p.m;
        const int stride = is_b ? p.stride_sfb : p.stride_sfa;
        rsrc_sf = make_rsrc(is_b ? sfb_e : sfa_e, (uint32_t)(rows - 1) * stride + (uint32_t)(p.k >> 5));
        voff_sf = min((is_b ? n0 : m0) + (wave & 3) * 64 + lane, rows - 1) * stride;
        rd_sfa = GEMM_LDS_BYTES + (wave_m * WAVE_M + r16) * 16;
        rd_sfb = GEMM_LDS_BYTES + BM * 16 + (wave_n * WAVE_N + r16) * 16;
    }
    auto issue_mx_group = [&](int group) {
        if constexpr (MODE == MODE_MX) {
            A8W8_LDS char* s = (A8W8_LDS char*)smem + GEMM_LDS_BYTES + (group & 1) * MX_GROUP_BYTES + wave * 1024;
            // the resource of the wave's matrix (waves 0-3 stage A rows, 4-7 B rows) is wave-uniform
            load_to_lds_16(rsrc_sf, s, voff_sf, group * 16);
        }
    };
    auto fetch_scales = [&](int kstep) {
        if constexpr (MODE == MODE_BLOCK) {
#pragma unroll
            for (int t = 0; t < TM; ++t)
                blk_sa_next[t] = sfa_f[(long long)kstep * p.stride_sfa + min(cm_base + 16 * t, p.m - 1)];
            const int nb = min(n0 + wave_n * WAVE_N, p.n - 1) >> 7;
            blk_sb_next = sfb_f[(long long)nb * p.stride_sfb + kstep];
        }
        if constexpr (MODE == MODE_MX) {
            // one dword per (row, K step) holds the four block exponents (four lanes reading one
            // dword is a broadcast); lane group g extracts byte g when the step begins, so that
            // nothing waits on these reads inside the step that issues them
            const char* s = smem + ((kstep >> 2) & 1) * MX_GROUP_BYTES + (kstep & 3) * 4;
#pragma unroll
            for (int t = 0; t < TM; ++t)
                mx_sa_next[t] = *(const int*)(s + rd_sfa + t * 256);
#pragma unroll
            for (int t = 0; t < TN; ++t)
                mx_sb_next[t] = *(const int*)(s + rd_sfb + t * 256);
        }
    };
    auto rotate_scales = [&]() {
        if constexpr (MODE == MODE_BLOCK) {
#pragma unroll
            for (int t = 0; t < TM; ++t) blk_sa[t] = blk_sa_next[t] * blk_sb_next;
        }
        if constexpr (MODE == MODE_MX) {
#pragma unroll
            for (int t = 0; t < TM; ++t) mx_sa[t] = (int)__builtin_amdgcn_ubfe((unsigned)mx_sa_next[t], 8 * g, 8);
#pragma unroll
            for (int t = 0; t < TN; ++t) mx_sb[t] = (int)__builtin_amdgcn_ubfe((unsigned)mx_sb_next[t], 8 * g, 8);
        }
    };

    issue_stage(0, 0);
    issue_mx_group(0);
    if constexpr (MODE == MODE_BLOCK) fetch_scales(0);
    __builtin_amdgcn_s_waitcnt(0);          // everything issued so far has landed
    __syncthreads();
    if constexpr (MODE == MODE_MX) fetch_scales(0);

    for (int ks = 0; ks < nk; ++ks) {
        const int cur = ks & 1;
        rotate_scales();
        if (ks + 1 < nk) {
            issue_stage(cur ^ 1, ks + 1);
            if ((ks & 3) == 0 && ks + 4 < nk) issue_mx_group((ks >> 2) + 1);
            fetch_scales(ks + 1);
        }

        // all A fragments of the step, B fragments one tile ahead of the MFMAs that use them
        v8i fa[TM], fb[2];
#pragma unroll
        for (int t = 0; t < TM; ++t) fa[t] = read_frag(cur, rd_a, t);
        fb[0] = read_frag(cur, rd_b, 0);
        if constexpr (MODE == MODE_BLOCK) {
            // Each 128-wide K step yields a partial tile that is rescaled into the running sum:
            // acc += part * (sfa * sfb).  The multiply-adds trail the MFMAs by BLK_LAG tiles so
            // that they never wait on a matrix-core result that is still in flight.
#ifndef A8W8_BLK_LAG
#define A8W8_BLK_LAG 4
#endif
            constexpr int BLK_LAG = A8W8_BLK_LAG;
            v4f part[BLK_LAG + 1];
#pragma unroll
            for (int t = 0; t < TM * TN + BLK_LAG; ++t) {
                if (t < TM * TN) {
                    const int j = t / TM, i = t % TM;
                    if (i == 0 && j + 1 < TN) fb[(j + 1) & 1] = read_frag(cur, rd_b, j + 1);
                    part[t % (BLK_LAG + 1)] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                        fb[j & 1], fa[i], v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);   // keep the lag: the scheduler would pull the FMAs up
                if (t >= BLK_LAG) {
                    const int u = t - BLK_LAG;
                    acc[u % TM][u / TM] += part[u % (BLK_LAG + 1)] * blk_sa[u % TM];
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if (j + 1 < TN) fb[(j + 1) & 1] = read_frag(cur, rd_b, j + 1);
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    if constexpr (MODE == MODE_MX) {
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                            fb[j & 1], fa[i], acc[i][j], 0, 0, 0, mx_sb[j], 0, mx_sa[i]);
                    } else {
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                            fb[j & 1], fa[i], acc[i][j], 0, 0, 0, 0, 0, 0);
                    }
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0);      // next stage has landed in LDS (this wave's part)
        __syncthreads();                    // ... everyone's part; and everyone is done reading `cur`
    }

    // ---- epilogue: dequantise in fp32, convert, store
    float sa[TM];
    float ts = 1.f;
    if constexpr (MODE == MODE_TENSOR) ts = sfa_f[0] * sfb_f[0];
    if constexpr (MODE == MODE_ROWCOL) {
#pragma unroll
        for (int i = 0; i < TM; ++i) sa[i] = sfa_f[min(cm_base + 16 * i, p.m - 1)];
    }
    char* c_base = (char*)p.c + (long long)batch * p.c_batch * (CDT == C_BF16 ? 2 : 4);
    const bool vec_ok = (CDT == C_BF16) ? ((p.ldc & 3) == 0 && (((uintptr_t)c_base) & 7) == 0)
                                        : ((p.ldc & 3) == 0 && (((uintptr_t)c_base) & 15) == 0);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int cn = cn_base + 16 * j;
        v4f sb = v4f{1.f, 1.f, 1.f, 1.f};
        if constexpr (MODE == MODE_ROWCOL) {
#pragma unroll
            for (int e = 0; e < 4; ++e) sb[e] = sfb_f[min(cn + e, p.n - 1)];
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int cm = cm_base + 16 * i;
            v4f v = acc[i][j];
            if constexpr (MODE == MODE_TENSOR) v *= ts;
            if constexpr (MODE == MODE_ROWCOL) v *= sb * sa[i];
            if (cm >= p.m) continue;
            if constexpr (CDT == C_BF16) {
                unsigned short* dst = (unsigned short*)c_base + (long long)cm * p.ldc + cn;
                if (vec_ok && cn + 3 < p.n) {
                    A8W8_STORE_C((v4u16*)dst, (v4u16{bf16_bits(v.x), bf16_bits(v.y), bf16_bits(v.z), bf16_bits(v.w)}));
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (cn + e < p.n) dst[e] = bf16_bits(v[e]);
                }
            } else {
                float* dst = (float*)c_base + (long long)cm * p.ldc + cn;
                if (vec_ok && cn + 3 < p.n) {
                    A8W8_STORE_C((v4f*)dst, v);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (cn + e < p.n) dst[e] = v[e];
                }
            }
        }
    }
}

}  // namespace a8w8
