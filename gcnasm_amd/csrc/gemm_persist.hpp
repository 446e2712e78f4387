// Persistent, software-pipelined dense A8W8 GEMM for gfx950, eight waves: block scales, row-major MX scales,
// and the per-tensor / row-col / bf16 cases with an odd number of K steps (the four-wave kernel of
// gemm_wide.hpp takes the even ones and tiled MX scales, gemm_small.hpp the problems of few tiles).
//
// Tile 256 x 256 x 128, 8 waves (4 along M x 2 along N), wave tile 64 x 128 = 4 x 8 MFMA
// tiles of 16 x 16 x 128, operands staged global -> LDS with 16-byte direct-to-LDS loads,
// two LDS stages of 64 KiB (laid out operand by operand: A of both stages, then B of both stages),
// 128-byte rows whose 16-byte slots are XOR-swizzled (see swz_key below).
//
// What differs from the plain kernel:
//  * One workgroup per CU walks a list of tiles; the K loop runs continuously across tile
//    boundaries, so the loads of the next tile's first K steps are already in flight while
//    the finished tile is scaled, converted and stored.
//  * An LDS stage is handed back in two parts.  After MFMA group 3 of a step every wave has
//    the step's A fragments and B tiles 0-3 in registers ("mid" barrier): the A half and the
//    low B half of the stage are free and the loads of the step after next start landing
//    there.  After group 6 all B tiles have been read ("end" barrier) and the high B half
//    follows.  Every byte therefore has about 1.5 K steps to arrive instead of one.
//  * The eight loads of a stage are issued one or two per MFMA group instead of as a burst,
//    and the next step's A fragments are fetched from LDS in the shadow of the last group.
//  * Barriers are raw s_barrier instructions with hand-placed s_waitcnt: the compiler's
//    workgroup fence would wait for every outstanding direct-to-LDS load at each barrier.
//    Loads complete in issue order, so "all but the newest four" (vmcnt(4)) at the end
//    barrier is exactly "the stage about to be read has landed".
#pragma once
#include <utility>

#include "gemm_common.hpp"

namespace a8w8 {

// LDS: two operand stages, then (MX only) two scale groups of 4 K steps.
constexpr int PERSIST_LDS_BYTES = GEMM_LDS_BYTES;
constexpr int PERSIST_LDS_BYTES_MX = GEMM_LDS_BYTES_MX;
// row/col mode: two buffers of 256 A-row + 256 B-row fp32 scales (the tile being multiplied and the
// one before it), filled by direct-to-LDS loads so that the epilogue waits on no global load
constexpr int ROWCOL_SCALE_BYTES = (BM + BN) * 4;
constexpr int PERSIST_LDS_BYTES_ROWCOL = GEMM_LDS_BYTES + 2 * ROWCOL_SCALE_BYTES;

// How many of the next step's four A fragments (plus the first B fragment) are fetched from LDS in
// the shadow of the current step's last MFMA group.  Bounded by the registers each mode has left:
// a spill inside the K loop is reloaded behind a wait for every load in flight.
#ifndef A8W8_NPF_ROWCOL
#define A8W8_NPF_ROWCOL 2
#endif
#ifndef A8W8_NPF_MX
#define A8W8_NPF_MX 1
#endif
#ifndef A8W8_NPF_BLOCK
#define A8W8_NPF_BLOCK 0
#endif
#define A8W8_PREFETCH_A(mode)                                                                        \
    ((mode) == MODE_TENSOR || (mode) == MODE_BF16 ? 4 : (mode) == MODE_ROWCOL ? A8W8_NPF_ROWCOL \
                                                     : (mode) == MODE_MX ? A8W8_NPF_MX : A8W8_NPF_BLOCK)
#ifndef A8W8_PERSIST_BLK_LAG
#define A8W8_PERSIST_BLK_LAG 4
#endif
#ifndef A8W8_BLK_SB
#define A8W8_BLK_SB 2
#endif
#if A8W8_BLK_SB == 1
#define A8W8_BLK_SCHED_BARRIER() __builtin_amdgcn_sched_barrier(0)
#elif A8W8_BLK_SB == 2
#define A8W8_BLK_SCHED_BARRIER() __builtin_amdgcn_sched_barrier(0x6)  /* VALU and SALU may cross */
#else
#define A8W8_BLK_SCHED_BARRIER() (void)0
#endif
#ifndef A8W8_PERSIST_SG
#define A8W8_PERSIST_SG 2
#endif
#ifndef A8W8_PERSIST_LINE_PAIRS
#define A8W8_PERSIST_LINE_PAIRS 1
#endif
#ifndef A8W8_PERSIST_LINES_BY_LANE
#define A8W8_PERSIST_LINES_BY_LANE 1      // 0: whole-line stores without the re-ordering of the lanes (measurement)
#endif
#ifndef A8W8_PERSIST_SB
#define A8W8_PERSIST_SB 0
#endif
#if A8W8_PERSIST_SB
#define A8W8_PERSIST_SCHED_BARRIER() __builtin_amdgcn_sched_barrier(0)
#else
#define A8W8_PERSIST_SCHED_BARRIER() (void)0
#endif

struct PersistParams {
    GemmParams g;
    int batch;        // work items = batch * tiles_m * tiles_n, walked with stride gridDim.x
    int items;
    TileMap map;      // item -> (batch entry, tile) without run-time divisors
};

template <int MODE, int CDT>
__global__ void __launch_bounds__(GEMM_THREADS, 1) gemm_a8w8_persist(PersistParams pp)
{
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const GemmParams& p = pp.g;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = wave_uniform(tid >> 6);
    const int wave_m = wave >> 1, wave_n = wave & 1;
    static_assert(MODE == MODE_TENSOR || MODE == MODE_ROWCOL || MODE == MODE_BLOCK || MODE == MODE_MX || MODE == MODE_BF16,
                  "tiled MX scales and MXFP4 operands run on the four-wave kernel");
    constexpr bool IS_MX = MODE == MODE_MX;
    constexpr int GROUP_SHIFT = 2;                                 // log2(K steps per scale group)
    constexpr int GROUP_MASK = (1 << GROUP_SHIFT) - 1;
    const int r16 = lane & 15, g = lane >> 4;
    const int nk = p.k / BK;                       // >= 2 (checked by the host)

    // ---------------------------------------------------------------- load side state
    // position of the stage whose loads are being issued: (item, k step), two steps ahead
    int ld_item = blockIdx.x, ld_ks = 0;
    const int groups_per_tile = (nk + GROUP_MASK) >> GROUP_SHIFT;   // MX scale groups per tile
    int ld_gbase = 0, cur_gbase = 0;                // running group count: picks the scale buffer
    __amdgpu_buffer_rsrc_t rsrc_a, rsrc_b, rsrc_sf;
    int ld_voff_a = 0, ld_voff_b = 0, voff_sf = 0;  // lane offsets of the operand and scale loads at the load position
    // LDS: [A of stage 0][A of stage 1][B of stage 0][B of stage 1], 32 KiB each: both stages of an
    // operand lie within 64 KiB of the lane's base address, so stage and tile offsets are immediates
    constexpr int HALF_STAGE = BM * BK, OPERAND_BYTES = 2 * HALF_STAGE;
    const int ld_row = wave * 8 + (lane >> 3);
    // lane i of a 1 KiB chunk lands on row (i>>3), slot (i&7) of the chunk's 8 rows; the slot holds
    // K-piece slot ^ key(row) with key(row) = (row & 7) ^ (((row >> 3) & 3) << 1), and bits 3-4 of the
    // tile row are (chunk & 3) = (wave & 3) for every chunk this wave fills
    const int ld_piece16 = ((lane & 7) ^ (((lane >> 3) ^ ((wave & 3) << 1)) & 7)) * 16;
    auto point_loads_at = [&](int item) __attribute__((always_inline)) {
        item = min(item, pp.items - 1);            // past the end: keep loading valid data nobody reads
        int batch, tm, tn;
        tile_of_item(pp.map, item, batch, tm, tn);
        const int m0 = tm * BM, n0 = tn * BN;
        rsrc_a = make_rsrc(p.a + (long long)batch * p.a_batch, (uint32_t)(p.m - 1) * p.lda + p.k);
        rsrc_b = make_rsrc(p.b + (long long)batch * p.b_batch, b_extent_bytes(p));
        ld_voff_a = (m0 + ld_row) * p.lda + ld_piece16;
        ld_voff_b = b_lane_offset(p, n0 + ld_row, ld_piece16);
        if constexpr (MODE == MODE_MX) {
            const bool is_b = wave >= 4;           // waves 0-3 stage A-row scales, 4-7 B-row scales
            const int rows = is_b ? p.n : p.m;
            const int stride = is_b ? p.stride_sfb : p.stride_sfa;
            const uint8_t* base = is_b ? (const uint8_t*)p.sfb + (long long)batch * p.sfb_batch
                                       : (const uint8_t*)p.sfa + (long long)batch * p.sfa_batch;
            rsrc_sf = make_rsrc(base, (uint32_t)(rows - 1) * stride + (uint32_t)(p.k >> 5));
            voff_sf = min((is_b ? n0 : m0) + (wave & 3) * 64 + lane, rows - 1) * stride;
        }
    };
    // one of the eight loads of a stage: 0..3 = A chunks, 4,5 = low B chunks, 6,7 = high B chunks.
    // Wave w fills rows 8w + 64j (+0..7) of each matrix; for B, j = 0, 2 are the rows of MFMA
    // tiles 0-3 of the two wave columns ("low"), j = 1, 3 those of tiles 4-7 ("high").
    auto issue_one = [&](int stage, int kstep, int which) __attribute__((always_inline)) {
        A8W8_LDS char* s = (A8W8_LDS char*)smem + stage * HALF_STAGE + wave * 1024;
        const int koff = kstep * BK;
        // One lane offset per operand (the wave's rows of the tile's first 64, set per tile); the 64-row
        // chunk rides in the scalar offset.  Rows past the end of a matrix are past the end of its
        // descriptor: they read as zero and only reach accumulators that are never stored.
        if (which < 4) {
            load_to_lds_16(rsrc_a, s + which * 8192, ld_voff_a, koff + 64 * which * p.lda);
        } else {
            const int j = which == 4 ? 0 : which == 5 ? 2 : which == 6 ? 1 : 3;
            load_to_lds_16(rsrc_b, s + OPERAND_BYTES + j * 8192, ld_voff_b, (kstep << p.b_kshift) + 64 * j * p.ldb);
        }
    };
    auto issue_mx_group = [&](int group) __attribute__((always_inline)) {
        if constexpr (IS_MX) {
            A8W8_LDS char* s =
                (A8W8_LDS char*)smem + GEMM_LDS_BYTES + ((ld_gbase + group) & 1) * MX_GROUP_BYTES + wave * 1024;
            load_to_lds_16(rsrc_sf, s, voff_sf, group * 16);   // 16 scale bytes per row and group
        }
    };
    int tile_seq = 0;                               // tiles this workgroup has started: picks the scale buffer
    auto issue_rowcol_scales = [&](int batch, int mm0, int nn0) __attribute__((always_inline)) {
        if constexpr (MODE == MODE_ROWCOL) {
            // thread t < 256 fetches sfa[m0 + t], the others sfb[n0 + t - 256] (row indices clamped)
            const bool is_b = wave >= 4;
            const int rows = is_b ? p.n : p.m;
            const float* base = is_b ? (const float*)p.sfb + (long long)batch * p.sfb_batch
                                     : (const float*)p.sfa + (long long)batch * p.sfa_batch;
            const __amdgpu_buffer_rsrc_t rs = make_rsrc(base, (uint32_t)rows * 4u);
            const int voff = min((is_b ? nn0 : mm0) + (wave & 3) * 64 + lane, rows - 1) * 4;
            A8W8_LDS char* s = (A8W8_LDS char*)smem + GEMM_LDS_BYTES + (tile_seq & 1) * ROWCOL_SCALE_BYTES + wave * 256;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, s, 4, voff, 0, 0, 0);
        }
    };
    auto advance_ld = [&]() __attribute__((always_inline)) {                      // the load position moves one K step
        if (++ld_ks == nk) {
            ld_ks = 0;
            ld_item += gridDim.x;
            ld_gbase += groups_per_tile;
            point_loads_at(ld_item);
        }
    };

    // ---------------------------------------------------------------- compute side state
    // LDS rows of the operands.  A: MFMA tile t, operand row r16 <- tile row 16t + r16.  B: the rows
    // of each 32-row group are dealt to a tile pair so that a lane ends up with eight consecutive n
    // (one 16-byte bf16 store, 64 contiguous bytes per C row and instruction):
    //     tile j, operand row 4g' + i  <-  row 32*(j/2) + 8g' + 4*(j%2) + i.
    // The swizzle key (row & 7) ^ (((row >> 3) & 3) << 1) keeps both read patterns free of LDS bank
    // conflicts (measured).  Only the tile's parity enters the key, the rest is an immediate offset.
    auto swz_key = [](int row) __attribute__((always_inline)) { return ((row & 7) ^ (((row >> 3) & 3) << 1)) & 7; };
    // For the rows of tile parity 1 the key differs from parity 0's in bit 2 only, and so do the two
    // K halves h of a fragment: slot(par, h) = slot(0, 0) ^ 4 (par ^ h).  Two address registers per
    // operand (h = 0, 1 of parity 0) therefore serve all four combinations; parity 1 swaps them and
    // adds its row offset as an immediate.
    constexpr int A_PAR_BYTES = 16 * BK, B_PAR_BYTES = 4 * BK;
    int rd_a[2], rd_b[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int row_b = 8 * (r16 >> 2) + (r16 & 3);
        const int row_a = r16;
        rd_a[h] = (wave_m * WAVE_M + row_a) * BK + ((((g + 4 * h) ^ swz_key(row_a)) & 7) << 4);
        rd_b[h] = OPERAND_BYTES + (wave_n * WAVE_N + row_b) * BK + ((((g + 4 * h) ^ swz_key(row_b)) & 7) << 4);
    }
    auto read_frag_at = [&](int stage, const int (&base)[2], int par, int byte_off) __attribute__((always_inline)) -> v8i {
        const char* s = smem + stage * HALF_STAGE + byte_off;
        const v4i lo = *(const v4i*)(s + base[par]);
        const v4i hi = *(const v4i*)(s + base[par ^ 1]);
        return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    };
    auto read_frag_a = [&](int stage, int t) __attribute__((always_inline)) -> v8i {
        return read_frag_at(stage, rd_a, t & 1, (t >> 1) * (32 * BK) + (t & 1) * A_PAR_BYTES);
    };
    auto read_frag_b = [&](int stage, int j) __attribute__((always_inline)) -> v8i {
        return read_frag_at(stage, rd_b, j & 1, (j >> 1) * (32 * BK) + (j & 1) * B_PAR_BYTES);
    };
    // MX scales (16 bytes per row per group of four K steps): B tile t at + (t >> 1) * 512 + (t & 1) * 64
    const int rd_sfa = GEMM_LDS_BYTES + (wave_m * WAVE_M + r16) * 16;
    const int rd_sfb = GEMM_LDS_BYTES + BM * 16 + (wave_n * WAVE_N + 8 * (r16 >> 2) + (r16 & 3)) * 16;

    int cur_item = blockIdx.x, cur_ks = 0;         // the step being multiplied
    int cur_batch = 0, m0 = 0, n0 = 0;
    auto point_compute_at = [&](int item) __attribute__((always_inline)) {
        int tm, tn;
        tile_of_item(pp.map, item, cur_batch, tm, tn);
        m0 = tm * BM;
        n0 = tn * BN;
    };

    v4f acc[TM][TN];
    auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
    };

    // scales consumed by the MFMAs of a step (BLOCK: fp32 per row x per column block, MX: E8M0 bytes)
    float blk_s[TM], blk_s_next[TM];
    int mx_sa[TM], mx_sb[TN], mx_sa_next[TM], mx_sb_next[TN];
    __amdgpu_buffer_rsrc_t blk_rs;                  // block scales of the tile whose scales are being fetched
    const float* blk_sfb_row = nullptr;
    int blk_voff[TM] = {0, 0, 0, 0};
    const int blk_sfa_step = p.stride_sfa * 4;
    auto point_block_scales_at = [&](int batch, int mm0, int nn0) __attribute__((always_inline)) {
        if constexpr (MODE == MODE_BLOCK) {
            const float* sfa_f = (const float*)p.sfa + (long long)batch * p.sfa_batch;
            const float* sfb_f = (const float*)p.sfb + (long long)batch * p.sfb_batch;
            blk_rs = make_rsrc(sfa_f, (uint32_t)((nk - 1) * p.stride_sfa + p.m) * 4u);
            const int nb = min(nn0 + wave_n * WAVE_N, p.n - 1) >> 7;
            blk_sfb_row = sfb_f + (long long)nb * p.stride_sfb;
            const int row0 = mm0 + wave_m * WAVE_M + r16;
#pragma unroll
            for (int t = 0; t < TM; ++t) blk_voff[t] = min(row0 + 16 * t, p.m - 1) * 4;
        }
    };
    auto fetch_step_scales = [&](int batch, int mm0, int nn0, int kstep, int gbase) __attribute__((always_inline)) {
        (void)gbase;
        if constexpr (MODE == MODE_BLOCK) {
            // A-row scales through a buffer descriptor (32-bit lane offsets instead of 64-bit pointers).
            // Descriptor, B-scale row and lane offsets change only with the tile: they are set up by
            // point_block_scales_at, so that a K step spends a handful of scalar instructions here.
            (void)batch; (void)mm0; (void)nn0;
            const float sb = blk_sfb_row[kstep];
#pragma unroll
            for (int t = 0; t < TM; ++t)
                blk_s_next[t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                              blk_rs, blk_voff[t], kstep * blk_sfa_step, 0)) * sb;
        }
        if constexpr (MODE == MODE_MX) {
            // one dword per (row, K step) holds the four block exponents; lane group g extracts
            // byte g when the step begins, so nothing waits on these reads in the step issuing them
            const char* s = smem + ((gbase + (kstep >> 2)) & 1) * MX_GROUP_BYTES + (kstep & 3) * 4;
#pragma unroll
            for (int t = 0; t < TM; ++t)
                mx_sa_next[t] = *(const int*)(s + rd_sfa + t * 256);
#pragma unroll
            for (int t = 0; t < TN; ++t)
                mx_sb_next[t] = *(const int*)(s + rd_sfb + (t >> 1) * 512 + (t & 1) * 64);
        }
    };
    auto rotate_step_scales = [&]() __attribute__((always_inline)) {
        if constexpr (MODE == MODE_BLOCK) {
#pragma unroll
            for (int t = 0; t < TM; ++t) blk_s[t] = blk_s_next[t];
        }
        if constexpr (MODE == MODE_MX) {
#pragma unroll
            for (int t = 0; t < TM; ++t) mx_sa[t] = (int)__builtin_amdgcn_ubfe((unsigned)mx_sa_next[t], 8 * g, 8);
#pragma unroll
            for (int t = 0; t < TN; ++t) mx_sb[t] = (int)__builtin_amdgcn_ubfe((unsigned)mx_sb_next[t], 8 * g, 8);
        }
    };

    // ---------------------------------------------------------------- epilogue of one tile
    auto store_tile = [&]() __attribute__((always_inline)) {
        const float* sfa_f = (const float*)p.sfa + (long long)cur_batch * p.sfa_batch;
        const float* sfb_f = (const float*)p.sfb + (long long)cur_batch * p.sfb_batch;
        const int cm_base = m0 + wave_m * WAVE_M + r16;
        auto cm_of = [&](int i) __attribute__((always_inline)) { return cm_base + 16 * i; };   // C row of MFMA tile i
        const int cn_base = n0 + wave_n * WAVE_N + 8 * g;      // + 32 * (tile pair): eight consecutive n
        float sa[TM];
        float ts = 1.f;
        if constexpr (MODE == MODE_TENSOR) ts = sfa_f[0] * sfb_f[0];
        char* c_base = (char*)p.c + (long long)cur_batch * p.c_batch * (CDT == C_BF16 ? 2 : 4);
        const bool vec_ok = (CDT == C_BF16) ? ((p.ldc & 7) == 0 && (((uintptr_t)c_base) & 15) == 0)
                                            : ((p.ldc & 3) == 0 && (((uintptr_t)c_base) & 15) == 0);
        // row/col scales were staged in LDS when the tile began (issue_rowcol_scales): reading them
        // waits on no global load, and a wait for a load issued after a store would also wait for
        // that store to be acknowledged (one counter, in issue order)
        float sb[TN / 2][8];
        if constexpr (MODE == MODE_ROWCOL) {
            const float* sc = (const float*)(smem + GEMM_LDS_BYTES + (tile_seq & 1) * ROWCOL_SCALE_BYTES);
#pragma unroll
            for (int i = 0; i < TM; ++i) sa[i] = sc[cm_of(i) - m0];
#pragma unroll
            for (int jp = 0; jp < TN / 2; ++jp) {
                const v4f lo = *(const v4f*)(sc + BM + (cn_base - n0) + 32 * jp), hi = *(const v4f*)(sc + BM + (cn_base - n0) + 32 * jp + 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) { sb[jp][e] = lo[e]; sb[jp][4 + e] = hi[e]; }
            }
        }
        // a tile that lies inside the matrix and takes 16-byte stores is written without per-lane checks (the
        // checked path spends more instructions on masks and branches than on stores)
        const bool whole = vec_ok && m0 + BM <= p.m && n0 + BN <= p.n;
        // such a tile goes out through a buffer descriptor over its own rows (store_c_16, store_c_lines), with 32-bit offsets
        constexpr int C_ES = CDT == C_BF16 ? 2 : 4;
        const __amdgpu_buffer_rsrc_t tile_rs =
            make_rsrc(c_base + ((long long)m0 * p.ldc + n0) * C_ES, (uint32_t)((BM - 1) * p.ldc + BN) * C_ES);
        // (unsigned arithmetic: with stride_c in the millions these byte offsets pass 2^31; the hardware takes them as unsigned)
        const uint32_t ldc_bytes = (uint32_t)p.ldc * C_ES;
        const int tile_row16 = (int)(16u * ldc_bytes);
        // bf16: one 16-byte store per piece, 64 contiguous bytes per row and instruction.  fp32: the lane's places in
        // the two stores of store_c_lines (rows 0 .. 7 / 8 .. 15 of the 16 rows of a piece)
        const int tile_lane_off = (int)((uint32_t)(wave_m * WAVE_M + r16) * ldc_bytes + (uint32_t)((wave_n * WAVE_N + 8 * g) * C_ES));
        const bool upper = r16 >= 8;
        int line_off_low, line_off_high;
        // (fp32: the two halves of a piece, 16 bytes apart; bf16: two pieces side by side, 64 bytes apart)
        constexpr bool BL = A8W8_PERSIST_LINES_BY_LANE != 0;
        // (worked out from an opaque copy of the lane number: values that depend on the lane alone would otherwise be computed
        // once, before the K loop, and held in registers the block-scale loop does not have: two of them spilled)
        int ln = lane;
        asm volatile("" : "+v"(ln));
        c_line_offsets<CDT == C_FP32 ? 16 : 64, BL>(ln, (int)((uint32_t)(wave_m * WAVE_M + c_line_row<BL>(ln)) * ldc_bytes),
                                                    (int)((uint32_t)(wave_m * WAVE_M + c_line_row<BL>(ln) + 8) * ldc_bytes), wave_n * WAVE_N * C_ES,
                                                    line_off_low, line_off_high);
        const int line_src_low = c_line_source<CDT == C_FP32 ? 16 : 64, BL>(ln, false), line_src_high = c_line_source<CDT == C_FP32 ? 16 : 64, BL>(ln, true);
        auto scaled_piece = [&](int i, int jp, float (&v)[8]) __attribute__((always_inline)) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                v[e] = acc[i][2 * jp + (e >> 2)][e & 3];
                if constexpr (MODE == MODE_TENSOR) v[e] *= ts;
                if constexpr (MODE == MODE_ROWCOL) v[e] *= sb[jp][e] * sa[i];
            }
        };
        auto packed_bf16 = [&](const float (&v)[8]) __attribute__((always_inline)) {
            v4i w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = bf16x2_bits(v[2 * e], v[2 * e + 1]);
            return w;
        };
        if (whole && CDT == C_BF16 && A8W8_PERSIST_LINE_PAIRS) {
            // bf16: the pieces of tile pairs 2 jpp and 2 jpp + 1 lie 64 bytes apart in every row; exchanged between the
            // lanes of rows r and r + 8 they leave as whole 128-byte lines, eight rows per store, which a compute unit
            // writes nearly twice as fast as 64-byte halves of sixteen rows
#pragma unroll
            for (int jpp = 0; jpp < TN / 4; ++jpp)
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    float v0[8], v1[8];
                    scaled_piece(i, 2 * jpp, v0);
                    scaled_piece(i, 2 * jpp + 1, v1);
                    store_c_lines<BL>(tile_rs, packed_bf16(v0), packed_bf16(v1), upper, line_src_low, line_src_high, line_off_low + 128 * jpp, line_off_high + 128 * jpp, i * tile_row16);
                }
            return;
        }
        if (whole) {
#pragma unroll
            for (int jp = 0; jp < TN / 2; ++jp)
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    float v[8];
                    scaled_piece(i, jp, v);
                    // 32 jp columns on (an immediate), 16 i rows down (a scalar)
                    if constexpr (CDT == C_BF16) {
                        store_c_16<true>(tile_rs, packed_bf16(v), tile_lane_off + 32 * jp * C_ES, i * tile_row16);
                    } else {
                        store_c_lines<BL>(tile_rs, __builtin_bit_cast(v4i, v4f{v[0], v[1], v[2], v[3]}),
                                      __builtin_bit_cast(v4i, v4f{v[4], v[5], v[6], v[7]}), upper, line_src_low, line_src_high, line_off_low + 32 * jp * C_ES,
                                      line_off_high + 32 * jp * C_ES, i * tile_row16);
                    }
                }
            return;
        }
#pragma unroll
        for (int jp = 0; jp < TN / 2; ++jp) {
            const int cn = cn_base + 32 * jp;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int cm = cm_of(i);
                float v[8];
                scaled_piece(i, jp, v);
                if (cm >= p.m) continue;
                if constexpr (CDT == C_BF16) {
                    unsigned short* dst = (unsigned short*)c_base + (long long)cm * p.ldc + cn;
                    if (vec_ok && cn + 7 < p.n) {
                        v4i w;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            w[e] = bf16x2_bits(v[2 * e], v[2 * e + 1]);
                        A8W8_STORE_C((v4i*)dst, w);
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (cn + e < p.n) dst[e] = bf16_bits(v[e]);
                    }
                } else {
                    float* dst = (float*)c_base + (long long)cm * p.ldc + cn;
                    if (vec_ok && cn + 7 < p.n) {
                        A8W8_STORE_C((v4f*)dst, (v4f{v[0], v[1], v[2], v[3]}));
                        A8W8_STORE_C((v4f*)(dst + 4), (v4f{v[4], v[5], v[6], v[7]}));
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (cn + e < p.n) dst[e] = v[e];
                    }
                }
            }
        }
    };

    // ---------------------------------------------------------------- prologue
    // The next step's A fragments and first B fragment are fetched in the shadow of the last MFMA
    // group; the block-scale mode has no registers to spare for that second set and reads them
    // when the step begins.
    constexpr int NPF = A8W8_PREFETCH_A(MODE);
    constexpr bool PREFETCH_FRAGS = NPF > 0;
    struct Frags {
        v8i a[TM];
        v8i b0;
    };
    Frags F[PREFETCH_FRAGS ? 2 : 1];
    const int my_items = (pp.items - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
    const int total_steps = my_items * nk;

    if (my_items == 0) return;
    point_loads_at(ld_item);
    point_compute_at(cur_item);
    // the stages of steps 0 and 1 in full and MX scale group 0; the load position stays at step 1,
    // whose last two loads the first step re-issues (same data, nobody is reading that stage yet)
#pragma unroll
    for (int w = 0; w < 8; ++w) issue_one(0, 0, w);
    issue_mx_group(0);
    advance_ld();
#pragma unroll
    for (int w = 0; w < 8; ++w) issue_one(1, ld_ks, w);
    if constexpr (MODE == MODE_BLOCK) {
        point_block_scales_at(cur_batch, m0, n0);
        fetch_step_scales(cur_batch, m0, n0, 0, 0);
    }
    issue_rowcol_scales(cur_batch, m0, n0);
    // vmcnt(8) lgkmcnt(0): step 0 (and MX scale group 0, issued before step 1's loads) has landed; the eight loads of
    // step 1 may still be on their way: the first step's end barrier waits for them like any other step's
    __builtin_amdgcn_s_waitcnt(0x0078);
    A8W8_RAW_BARRIER();
    if constexpr (IS_MX) fetch_step_scales(cur_batch, m0, n0, 0, 0);
    if constexpr (PREFETCH_FRAGS) {
#pragma unroll
        for (int t = 0; t < NPF; ++t) F[0].a[t] = read_frag_a(0, t);
        F[0].b0 = read_frag_b(0, 0);
    }
    zero_acc();

    // ---------------------------------------------------------------- one K step
    // Loads of the stage at the load position X: A chunks after MFMA groups 3..6 of step X-2,
    // first low/high B chunks after group 7, the second ones after groups 0 and 1 of step X-1;
    // the position advances after group 2.
    auto step = [&](auto parity) __attribute__((always_inline)) {
        constexpr int P = decltype(parity)::value;
        Frags& cur = F[PREFETCH_FRAGS ? P : 0];
        Frags& nxt = F[PREFETCH_FRAGS ? P ^ 1 : 0];
        rotate_step_scales();
#pragma unroll
        for (int t = NPF; t < TM; ++t) cur.a[t] = read_frag_a(P, t);
        if constexpr (!PREFETCH_FRAGS) cur.b0 = read_frag_b(P, 0);
        // where the next step lives (it may be the first step of this workgroup's next tile)
        const bool last_of_tile = cur_ks + 1 == nk;
        int nx_batch = cur_batch, nx_m0 = m0, nx_n0 = n0, nx_gbase = cur_gbase;
        const int nx_ks = last_of_tile ? 0 : cur_ks + 1;
        if (last_of_tile) {
            const int item = min(cur_item + (int)gridDim.x, pp.items - 1);
            int tm, tn;
            tile_of_item(pp.map, item, nx_batch, tm, tn);
            nx_m0 = tm * BM;
            nx_n0 = tn * BN;
            nx_gbase = cur_gbase + groups_per_tile;
            point_block_scales_at(nx_batch, nx_m0, nx_n0);   // the fetch at group 2 is for the next tile's step 0
        }

        v8i fb[TN];
        fb[0] = cur.b0;
        // block scales: acc += part * scale trails the MFMA that made `part` by BLK_LAG tiles
        constexpr int BLK_LAG = A8W8_PERSIST_BLK_LAG;
        v4f part[BLK_LAG + 1];
        (void)part;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            if (j + 1 < TN) fb[j + 1] = read_frag_b(P, j + 1);
            A8W8_PERSIST_SCHED_BARRIER();
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                if constexpr (MODE == MODE_MX) {
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[j], cur.a[i], acc[i][j], 0, 0, 0,
                                                                                 mx_sb[j], 0, mx_sa[i]);
                } else if constexpr (MODE == MODE_BLOCK) {
                    const int t = j * TM + i;
                    part[t % (BLK_LAG + 1)] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                        fb[j], cur.a[i], v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                    A8W8_BLK_SCHED_BARRIER();
                    if (t >= BLK_LAG) {
                        const int u = t - BLK_LAG;
                        acc[u % TM][u / TM] += part[u % (BLK_LAG + 1)] * blk_s[u % TM];
                    }
                    A8W8_BLK_SCHED_BARRIER();
                    if (t == TM * TN - 1) {
#pragma unroll
                        for (int u = TM * TN - BLK_LAG; u < TM * TN; ++u)
                            acc[u % TM][u / TM] += part[u % (BLK_LAG + 1)] * blk_s[u % TM];
                    }
                } else if constexpr (MODE == MODE_BF16) {
                    // a 128-byte row is 64 bf16: the fragment's two 16-byte halves feed one 16x16x32 MFMA each
                    // (both operands split K the same way, so the order inside an instruction is immaterial).
                    // First halves here, second halves after the loop: back-to-back MFMAs on one accumulator stall.
                    const v4i blo = {fb[j][0], fb[j][1], fb[j][2], fb[j][3]};
                    const v4i alo = {cur.a[i][0], cur.a[i][1], cur.a[i][2], cur.a[i][3]};
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, blo), __builtin_bit_cast(v8bf, alo),
                                                                        acc[i][j], 0, 0, 0);
                } else {
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[j], cur.a[i], acc[i][j], 0, 0, 0,
                                                                                 0, 0, 0);
                }
            }
            if constexpr (MODE == MODE_BF16) {
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    const v4i bhi = {fb[j][4], fb[j][5], fb[j][6], fb[j][7]};
                    const v4i ahi = {cur.a[i][4], cur.a[i][5], cur.a[i][6], cur.a[i][7]};
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, bhi), __builtin_bit_cast(v8bf, ahi),
                                                                        acc[i][j], 0, 0, 0);
                }
            }
            A8W8_PERSIST_SCHED_BARRIER();
#if A8W8_PERSIST_SG
            if constexpr (MODE != MODE_BLOCK) {
                // spread the two LDS reads of the next B fragment between this group's MFMAs
                constexpr int MPF = MODE == MODE_BF16 ? 2 : 1;      // MFMAs per operand fragment pair
                if (j + 1 < TN) {
                    __builtin_amdgcn_sched_group_barrier(0x008, MPF, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, MPF, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 2 * MPF, 0);
                } else if (A8W8_PERSIST_SG >= 2 && PREFETCH_FRAGS) {
                    // the last group runs beside the next step's prefetched fragments
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        __builtin_amdgcn_sched_group_barrier(0x008, MPF, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, (2 * NPF + 2 + 3) / 4, 0);
                    }
                }
            }
#endif

            if (j == 0) issue_one(P ^ 1, ld_ks, 5);
            if (j == 1) issue_one(P ^ 1, ld_ks, 7);
            if (j == 2) {
                advance_ld();
                if constexpr (IS_MX) {
                    if ((ld_ks & GROUP_MASK) == 0) issue_mx_group(ld_ks >> GROUP_SHIFT);   // scales of the group starting at ld_ks
                }
                if constexpr (MODE == MODE_BLOCK) fetch_step_scales(nx_batch, nx_m0, nx_n0, nx_ks, 0);
            }
            if (j == 3) {
                __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): A fragments and B tiles 0..4 are in registers
                A8W8_RAW_BARRIER();                   // mid: the A half and low B half of stage P are free
                issue_one(P, ld_ks, 0);
            }
            if (j == 4) issue_one(P, ld_ks, 1);
            if (j == 5) issue_one(P, ld_ks, 2);
            if (j == 6) {
                issue_one(P, ld_ks, 3);
                __builtin_amdgcn_s_waitcnt(0x0074);   // vmcnt(4) lgkmcnt(0): the next stage has landed
                A8W8_RAW_BARRIER();                   // end: all of stage P is free
                if constexpr (PREFETCH_FRAGS) {
#pragma unroll
                    for (int t = 0; t < NPF; ++t) nxt.a[t] = read_frag_a(P ^ 1, t);
                    nxt.b0 = read_frag_b(P ^ 1, 0);
                }
                if constexpr (MODE == MODE_MX) fetch_step_scales(nx_batch, nx_m0, nx_n0, nx_ks, nx_gbase);
            }
            if (j == 7) {
                issue_one(P, ld_ks, 4);
                issue_one(P, ld_ks, 6);
            }
        }
        if (last_of_tile) {
            store_tile();
            zero_acc();
            cur_item += gridDim.x;
            cur_ks = 0;
            cur_batch = nx_batch;
            m0 = nx_m0;
            n0 = nx_n0;
            cur_gbase = nx_gbase;
            if constexpr (MODE == MODE_ROWCOL) ++tile_seq;
            // the next tile's row/col scales: in flight from here, landed (and past a barrier) long
            // before its epilogue; the end barrier's "all but the newest four loads" covers it
            issue_rowcol_scales(cur_batch, m0, n0);
        } else {
            ++cur_ks;
        }
    };

    for (int s = 0; s < total_steps; s += 2) {
        step(std::integral_constant<int, 0>{});
        if (s + 1 < total_steps) step(std::integral_constant<int, 1>{});
    }
    __builtin_amdgcn_s_waitcnt(0);   // no direct-to-LDS load may outlive the workgroup's LDS allocation
}

}  // namespace a8w8
