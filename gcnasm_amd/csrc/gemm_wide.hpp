// Persistent dense A8W8 GEMM for gfx950 with four waves per workgroup and both operand fragment
// sets resident in registers.
//
// Tile 256 x 256 x 128, 4 waves (2 along M x 2 along N), wave tile 128 x 128 = 8 x 8 MFMA tiles of
// 16 x 16 x 128: 256 accumulator registers per lane and 16 operand fragments (128 registers).  Each
// fragment is read from LDS once per K step, so a step moves 128 KiB out of LDS instead of the 192 KiB
// of the eight-wave 64 x 128 layout; with one wave per SIMD nothing else hides an LDS wait, so the
// schedule below never has one:
//
//  * A K step is four quadrants of 16 MFMAs: (aL,bL) (aL,bH) (aH,bH) (aH,bL) on even steps and
//    (aL,bH) (aL,bL) (aH,bL) (aH,bH) on odd ones, where aL/aH are the fragments of the wave's A rows
//    0-63 / 64-127 and bL/bH the same for B.  Consecutive quadrants share one set, so exactly one
//    set of four fragments dies per quadrant; it is re-read (8 ds_read_b128, for the same step or the
//    next one) while the quadrant after its death runs and is first used one quadrant later.
//  * Seen from LDS, a quadrant reads one quarter of a stage (16 KiB: 64 + 64 rows of one operand, the
//    same for all four waves).  Two barriers per step ("mid" after the second quadrant, "end" after
//    the fourth) hand the two quarters read since the last barrier back to the loads, and each
//    quadrant issues one quarter (four 1 KiB direct-to-LDS loads per wave) of the step after next.
//    Every byte has 1.5 K steps to arrive.
//  * Loads complete in issue order: "all but the newest 16" at a barrier is "the two quarters the
//    next two quadrants read have landed".
#pragma once
#include <type_traits>
#include <utility>

#include "gemm_persist.hpp"

// Measurement switches (all off in the library that ships): each removes one ingredient of the K loop so that its
// cost can be read off a timing of the same launch.  The results of an ablated build are wrong by construction.
//   A8W8_ABLATE_OPERAND_LOADS   the loop issues no A/B loads (the two stages keep what the prologue brought)
//   A8W8_ABLATE_SCALE_LOADS     tiled MX: no scale bytes are fetched after the first batch
//   A8W8_ABLATE_HOT_SCALES      tiled MX: every batch re-reads the tile's first batch (lines that are already in L2)
//   A8W8_ABLATE_SCALE_READS     tiled MX: the scale registers are not refreshed from LDS
//   A8W8_ABLATE_UNSCALED_MFMA   tiled MX: the plain form of the MFMA in place of the scaled one
//   A8W8_ABLATE_STORES          whole tiles are neither converted nor written (the accumulators are still read out)
//   A8W8_ABLATE_STORE_INSTRUCTIONS   whole tiles are read out and converted, only the 16-byte store instructions are left out
//                               (store_c_16 in a8w8_device.hpp: every kernel's whole-tile stores)
// and three that keep the results right:
//   A8W8_WIDE_WRITE_THROUGH=0   bf16 tiles are stored write-back instead of written through
//   A8W8_WIDE_BURST=0           the tile is written out in pieces among the MFMAs of its last K step and of the next
//                               tile's first quadrant, instead of in one burst between the two steps
//   A8W8_WIDE_LINE_PAIRS=0      bf16 tiles go out as 64-byte pieces of sixteen rows per store instead of whole lines of eight
//   A8W8_WIDE_LINES_BY_LANE=1   the whole-line stores' 16-byte units are moved between the lanes so that consecutive lanes write
//                               consecutive bytes (store_c_lines in a8w8_device.hpp; what the eight-wave kernel does)
//   A8W8_WIDE_READS_EARLY=0     a quadrant's LDS reads follow every second MFMA to its end instead of its first eight
//   A8W8_WIDE_STAGGER=n         workgroups start up to 7 n 64 clocks apart
#if defined(A8W8_ABLATE_OPERAND_LOADS) || defined(A8W8_ABLATE_SCALE_LOADS) || defined(A8W8_ABLATE_HOT_SCALES) || \
    defined(A8W8_ABLATE_SCALE_READS) || defined(A8W8_ABLATE_UNSCALED_MFMA) || defined(A8W8_ABLATE_STORES) || \
    defined(A8W8_ABLATE_STORE_INSTRUCTIONS)
#define A8W8_ABLATED 1
#else
#define A8W8_ABLATED 0
#endif

#ifndef A8W8_WIDE_WRITE_THROUGH
#define A8W8_WIDE_WRITE_THROUGH 1
#endif
#ifndef A8W8_WIDE_BURST
#define A8W8_WIDE_BURST 1
#endif
#ifndef A8W8_WIDE_LINE_PAIRS
#define A8W8_WIDE_LINE_PAIRS 1
#endif
#ifndef A8W8_WIDE_LINES_BY_LANE
#define A8W8_WIDE_LINES_BY_LANE 0
#endif
#ifndef A8W8_WIDE_READS_EARLY
#define A8W8_WIDE_READS_EARLY 1
#endif

namespace a8w8 {

constexpr int WIDE_THREADS = 256;
constexpr int WIDE_T = 8;                            // 8 x 8 MFMA tiles per wave
constexpr int wide_lds_bytes(int mode)
{
    // tiled MX scales: two buffers of two scale groups each, i.e. all of the 160 KiB
    return GEMM_LDS_BYTES + ((mode == MODE_MXT || mode == MODE_F4T) ? 4 * MX_GROUP_BYTES : mode == MODE_ROWCOL ? 2 * ROWCOL_SCALE_BYTES : 0);
}

// The 64 accumulator tiles of a wave live in accumulator registers a[0:255], tile (i, j) in
// a[4 (8i + j) : +3].  They are named in assembly statements only and never appear as variables: the
// compiler allocates nothing there (its own registers stay below 256, which the build checks), so no
// copy, spill or re-materialisation can come between two MFMAs of one tile.  The statements keep
// their order; the compiler does not see the MFMAs' latency, so the code that reads an accumulator
// makes sure that enough instructions separate it from the last MFMA into that tile.
template <int N, class F, int... I>
A8W8_DEV void static_for_impl(F&& f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
A8W8_DEV void static_for(F&& f)
{
    static_for_impl<N>(f, std::make_integer_sequence<int, N>{});
}

// tile LO/4 += a . b, or = a . b when ZC (the tile's first K step)
template <int LO, bool ZC>
A8W8_DEV void mfma_acc(const v8i& a, const v8i& b)
{
    if constexpr (ZC) asm volatile("v_mfma_f32_16x16x128_f8f6f4 a[%2:%3], %0, %1, 0" ::"v"(a), "v"(b), "n"(LO), "n"(LO + 3));
    else asm volatile("v_mfma_f32_16x16x128_f8f6f4 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(a), "v"(b), "n"(LO), "n"(LO + 3));
}
// the same with E8M0 block scales: byte OA of sa scales a's K block of the lane, byte OB of sb b's
template <int LO, bool ZC, int OA, int OB>
A8W8_DEV void mfma_acc_mx(const v8i& a, const v8i& b, int sa, int sb)
{
    if constexpr (ZC)
        asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[%4:%5], %0, %1, 0, %2, %3 op_sel:[%6,%7,0] op_sel_hi:[%8,%9,0]" ::"v"(a),
                     "v"(b), "v"(sa), "v"(sb), "n"(LO), "n"(LO + 3), "n"(OA & 1), "n"(OB & 1), "n"(OA >> 1), "n"(OB >> 1));
    else
        asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[%4:%5], %0, %1, a[%4:%5], %2, %3 op_sel:[%6,%7,0] op_sel_hi:[%8,%9,0]" ::"v"(a),
                     "v"(b), "v"(sa), "v"(sb), "n"(LO), "n"(LO + 3), "n"(OA & 1), "n"(OB & 1), "n"(OA >> 1), "n"(OB >> 1));
}
// bf16 operands: one 16 x 16 x 32 MFMA per 16-byte half of a fragment
template <int LO, bool ZC>
A8W8_DEV void mfma_acc_bf16(const v4i& a, const v4i& b)
{
    if constexpr (ZC) asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, 0" ::"v"(a), "v"(b), "n"(LO), "n"(LO + 3));
    else asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(a), "v"(b), "n"(LO), "n"(LO + 3));
}
// packed E2M1 operands (format 4 for both): one 16 x 16 x 128 MFMA per 16-byte half of a fragment
template <int LO, bool ZC, int OA, int OB>
A8W8_DEV void mfma_acc_f4(const v4i& a, const v4i& b, int sa, int sb)
{
    if constexpr (ZC)
        asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[%4:%5], %0, %1, 0, %2, %3 op_sel:[%6,%7,0] op_sel_hi:[%8,%9,0] cbsz:4 blgp:4" ::"v"(a),
                     "v"(b), "v"(sa), "v"(sb), "n"(LO), "n"(LO + 3), "n"(OA & 1), "n"(OB & 1), "n"(OA >> 1), "n"(OB >> 1));
    else
        asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[%4:%5], %0, %1, a[%4:%5], %2, %3 op_sel:[%6,%7,0] op_sel_hi:[%8,%9,0] cbsz:4 blgp:4" ::"v"(a),
                     "v"(b), "v"(sa), "v"(sb), "n"(LO), "n"(LO + 3), "n"(OA & 1), "n"(OB & 1), "n"(OA >> 1), "n"(OB >> 1));
}
template <int IDX>
A8W8_DEV float acc_read()
{
    float x;
    asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(IDX));
    return x;
}

template <int MODE, int CDT>
__global__ void __launch_bounds__(WIDE_THREADS) __attribute__((amdgpu_waves_per_eu(1, 1)))
gemm_a8w8_wide(PersistParams pp)
{
    static_assert(MODE == MODE_TENSOR || MODE == MODE_ROWCOL || MODE == MODE_MXT || MODE == MODE_BF16 || MODE == MODE_F4T,
                  "modes of the four-wave kernel");
    // MODE_F4T (packed E2M1 operands): a 128-byte K step holds 256 elements = eight scale blocks = one
    // "pair of K steps" of the tiled scale layout: the tiled-MX plumbing serves it with a scale fetch
    // every step and two 16 x 16 x 128 FP4 MFMAs per fragment pair.  MODE_BF16: a step is 64 elements,
    // two 16 x 16 x 32 MFMAs per fragment pair, no scales.
    constexpr bool IS_MXT = MODE == MODE_MXT || MODE == MODE_F4T;   // tiled E8M0 scales
    constexpr int MPF = (MODE == MODE_BF16 || MODE == MODE_F4T) ? 2 : 1;     // MFMAs per fragment pair
    constexpr int PAIR_STEPS = MODE == MODE_F4T ? 1 : 2;             // K steps served by one fetch of scales
    // tiled MX scales are laid out for A tiles whose rows are dealt like the B tiles' rows
    constexpr bool PERM_A = IS_MXT;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    // all 256 accumulator registers are in use (this is what sizes the wave's register allocation)
    asm volatile("" ::: "a0", "a255");
    const GemmParams& p = pp.g;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = wave_uniform(tid >> 6);
    const int wave_m = wave >> 1, wave_n = wave & 1;
    const int r16 = lane & 15, g = lane >> 4;
    const int nk = p.k / BK;                       // >= 2 (checked by the host)

    // LDS: [A of stage 0][A of stage 1][B of stage 0][B of stage 1], 32 KiB each.  A lane's read
    // addresses are its row and K-piece offset inside an operand (below 32 KiB) plus the stage and the
    // fragment's tile offset; keeping both stages of an operand within 64 KiB makes the latter two an
    // instruction immediate, so two address registers per operand serve every read.
    constexpr int HALF_STAGE = BM * BK;             // one operand of one stage
    constexpr int OPERAND_BYTES = 2 * HALF_STAGE;   // both stages of one operand

    // ---------------------------------------------------------------- load side
    int ld_item = blockIdx.x, ld_ks = 0;           // the step whose quarters are being issued
    __amdgpu_buffer_rsrc_t rsrc_a, rsrc_b;
    const int ld_row = wave * 8 + (lane >> 3);
    // lane i of a 1 KiB load lands on row (i >> 3), slot (i & 7) of 8 consecutive tile rows; the slot
    // holds K piece slot ^ key(row), key(row) = (row & 7) ^ (((row >> 3) & 3) << 1), and bits 3-4 of
    // the tile row equal the wave number for every load this wave issues
    const int ld_piece16 = ((lane & 7) ^ (((lane >> 3) ^ (wave << 1)) & 7)) * 16;
    // A load's address is lane offset + scalar offset: the lane part (two row groups of the tile per
    // operand) changes only with the tile, the scalar part is the K step plus a multiple of the row
    // stride.  Rows past the end of a matrix are past the end of its descriptor: they read
    // as zero and only reach accumulators that are never stored.
    int ld_voff_a[2] = {0, 0}, ld_voff_b[2] = {0, 0};   // rows 8w.. and 128 + 8w.. of the tile
    auto point_loads_at = [&](int item) __attribute__((always_inline)) {
        item = min(item, pp.items - 1);            // past the end: keep loading valid data nobody reads
        int batch, tm, tn;
        tile_of_item(pp.map, item, batch, tm, tn);
        rsrc_a = make_rsrc(p.a + (long long)batch * p.a_batch, (uint32_t)(p.m - 1) * p.lda + p.k);
        rsrc_b = make_rsrc(p.b + (long long)batch * p.b_batch, b_extent_bytes(p));
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            ld_voff_a[h] = (tm * BM + 128 * h + ld_row) * p.lda + ld_piece16;
            ld_voff_b[h] = b_lane_offset(p, tn * BN + 128 * h + ld_row, ld_piece16);
        }
    };
    // Load l (0..3) of quarter qt (0 aL, 1 aH, 2 bL, 3 bH) of the step at the load position.  A quarter
    // is tile rows [64h, 64h + 64) and [128 + 64h, 192 + 64h) of one operand (h = qt & 1): the L or H
    // rows of both wave rows (A) or wave columns (B).  Wave w fills rows 8w.. and 32 + 8w.. of each.
    int wave_lds = wave * 1024;
    auto issue_one = [&](int stage, int qt, int l) __attribute__((always_inline)) {
        const int row0 = 128 * (l >> 1) + 64 * (qt & 1) + 32 * (l & 1);
        A8W8_LDS char* s = (A8W8_LDS char*)smem + ((qt >= 2 ? OPERAND_BYTES : 0) + stage * HALF_STAGE + row0 * BK) + wave_lds;
        // four scalar offsets per operand and step (K step + 0, 32, 64 or 96 rows), each used twice
        const int rows = 64 * (qt & 1) + 32 * (l & 1);
        if (qt < 2) load_to_lds_16(rsrc_a, s, ld_voff_a[l >> 1], ld_ks * BK + rows * p.lda);
        else load_to_lds_16(rsrc_b, s, ld_voff_b[l >> 1], (ld_ks << p.b_kshift) + rows * p.ldb);
    };
    auto advance_ld = [&]() __attribute__((always_inline)) {
        if (++ld_ks == nk) {
            ld_ks = 0;
            ld_item += gridDim.x;
            point_loads_at(ld_item);
        }
    };

    // Tiled MX scales: the exponents of a 64-row block for four K steps are 1 KiB of contiguous memory
    // in the order the lanes read them ([pair of steps][lane (r16, g)][8 bytes]).  Wave w copies block w
    // of the A tile and block w of the B tile of one scale group into LDS buffer `buf`.  Everything
    // that depends on the tile (batch entry, first block of the tile) is worked out once per tile, for
    // this tile and the next one, so that a group costs two loads and a few scalar instructions.
    struct ScaleTile {
        const uint8_t* base[2];                    // scale arrays of the tile's batch entry (A side, B side)
        int blk[2];                                // the tile's first 64-row block
    };
    ScaleTile sf_cur = {}, sf_next = {};
    const int sf_nblk[2] = {(p.m + 63) >> 6, (p.n + 63) >> 6};
    const uint32_t sf_bytes[2] = {(uint32_t)mx_tiled_bytes(p.m, MODE == MODE_F4T ? 2 * p.k : p.k),
                                  (uint32_t)mx_tiled_bytes(p.n, MODE == MODE_F4T ? 2 * p.k : p.k)};
    auto point_scales_at = [&](ScaleTile& t, int item) __attribute__((always_inline)) {
        if constexpr (IS_MXT) {
            item = min(item, pp.items - 1);
            int batch, tm, tn;
            tile_of_item(pp.map, item, batch, tm, tn);
            t.base[0] = (const uint8_t*)p.sfa + (long long)batch * p.sfa_batch;
            t.base[1] = (const uint8_t*)p.sfb + (long long)batch * p.sfb_batch;
            t.blk[0] = tm * (BM / 64);
            t.blk[1] = tn * (BN / 64);
        }
    };
    const int lane16 = lane * 16;
    // The scale loads are few but slow (each touches lines that are cold in L2; measured: the same
    // loads from an always-hot region make the 8192^3 launch 10% faster on all-zero operands and 3% on
    // random ones).  They are issued in batches of GPB scale groups, as rarely as LDS allows.
    constexpr int GPB = 2;
    constexpr int BATCH_BYTES = GPB * MX_GROUP_BYTES;
    auto issue_mx_batch = [&](const ScaleTile& t, int batch, int buf) __attribute__((always_inline)) {
        if constexpr (IS_MXT) {
#pragma unroll
            for (int gi = 0; gi < GPB; ++gi)
#pragma unroll
                for (int side = 0; side < 2; ++side) {
                    const __amdgpu_buffer_rsrc_t rs = make_rsrc(t.base[side], sf_bytes[side]);   // past the end: reads 0
                    A8W8_LDS char* s =
                        (A8W8_LDS char*)smem + GEMM_LDS_BYTES + buf * BATCH_BYTES + gi * MX_GROUP_BYTES + side * 4096 + wave_lds;
                    load_to_lds_16(rs, s, lane16, ((batch * GPB + gi) * sf_nblk[side] + t.blk[side] + wave) * 1024);
                }
        }
    };
    // Row/col scales of a tile: thread t fetches sfa[m0 + t] and sfb[n0 + t] (indices clamped) into LDS
    // buffer `buf`, so that the epilogue waits on no global load.
    auto issue_rowcol_scales = [&](int batch, int mm0, int nn0, int buf) __attribute__((always_inline)) {
        if constexpr (MODE == MODE_ROWCOL) {
#pragma unroll
            for (int side = 0; side < 2; ++side) {
                const int rows = side ? p.n : p.m;
                const float* base = side ? (const float*)p.sfb + (long long)batch * p.sfb_batch
                                         : (const float*)p.sfa + (long long)batch * p.sfa_batch;
                const __amdgpu_buffer_rsrc_t rs = make_rsrc(base, (uint32_t)rows * 4u);
                const int voff = min((side ? nn0 : mm0) + tid, rows - 1) * 4;
                A8W8_LDS char* s = (A8W8_LDS char*)smem + GEMM_LDS_BYTES + buf * ROWCOL_SCALE_BYTES + side * (BM * 4) + wave * 256;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, s, 4, voff, 0, 0, 0);
            }
        }
    };

    // ---------------------------------------------------------------- compute side
    // LDS rows as in the eight-wave kernel.  A: MFMA tile t, operand row r16 <- wave row 16t + r16.
    // B: tile j, operand row 4g' + i <- wave row 32 (j/2) + 8g' + 4 (j%2) + i, so that a lane ends up
    // with eight consecutive n.  For tile parity 1 the swizzle key differs from parity 0's in bit 2
    // only, as do the two K halves h of a fragment: two address registers per operand serve all four.
    auto swz_key = [](int row) __attribute__((always_inline)) { return ((row & 7) ^ (((row >> 3) & 3) << 1)) & 7; };
    constexpr int A_PAR_BYTES = (PERM_A ? 4 : 16) * BK, B_PAR_BYTES = 4 * BK;
    int rd_a[2], rd_b[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int row_b = 8 * (r16 >> 2) + (r16 & 3);
        const int row_a = PERM_A ? row_b : r16;
        rd_a[h] = (wave_m * 128 + row_a) * BK + ((((g + 4 * h) ^ swz_key(row_a)) & 7) << 4);
        rd_b[h] = OPERAND_BYTES + (wave_n * 128 + row_b) * BK + ((((g + 4 * h) ^ swz_key(row_b)) & 7) << 4);
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

    // MX scales in registers: per 64-row block of the wave's A rows (and B rows) one dword per tile
    // pair, whose byte 2 (tile parity) + (step parity) belongs to the MFMA; they serve two K steps.
    const int lane_rg = r16 * 4 + g;
    const int rd_sfa = GEMM_LDS_BYTES + wave_m * 2048 + lane_rg * 8;
    const int rd_sfb = GEMM_LDS_BYTES + 4096 + wave_n * 2048 + lane_rg * 8;
    v2i sc_a[2], sc_b[2], sc_a_next[2], sc_b_next[2];
    int sc_rd_off = 0;                              // LDS offset (buffer, pair) of the scales to fetch next
    constexpr int BATCH_STEPS = 2 * 2 * PAIR_STEPS;  // K steps served by one batch: two scale groups of two pairs
    const int batches_per_tile = (nk + BATCH_STEPS - 1) / BATCH_STEPS;
    int cur_bbase = 0;                              // running batch count: picks the scale buffer

    int cur_item = blockIdx.x;                     // the tile being multiplied
    int cur_batch = 0, m0 = 0, n0 = 0;
    auto point_compute_at = [&](int item) __attribute__((always_inline)) {
        item = min(item, pp.items - 1);
        int tm, tn;
        tile_of_item(pp.map, item, cur_batch, tm, tn);
        m0 = tm * BM;
        n0 = tn * BN;
    };

    // ---------------------------------------------------------------- epilogue, in pieces
    // The tile whose accumulators are being written out (the current one until its last K step has
    // begun, then it stays while the next tile's first step runs).
    int ep_batch = 0, ep_m0 = 0, ep_n0 = 0, ep_seq = 0;
    int tile_seq = 0;                               // tiles this workgroup has started: picks the row/col scale buffer
    float ep_ts = 1.f;
    bool ep_vec_ok = false;                         // C rows of this batch entry take 16-byte stores
    // whole tiles go out through a buffer descriptor over the tile's own rows (store_c_16)
    __amdgpu_buffer_rsrc_t ep_rs;
    int ep_lane_off = 0, ep_row_bytes = 0;
    // whose 16 bytes the lane writes in the two stores of store_c_lines (itself unless the lanes are re-ordered)
    const int ep_line_src_low = c_line_source<CDT == C_FP32 ? 16 : 64, A8W8_WIDE_LINES_BY_LANE != 0>(lane, false);
    const int ep_line_src_high = c_line_source<CDT == C_FP32 ? 16 : 64, A8W8_WIDE_LINES_BY_LANE != 0>(lane, true);
    int ep_line_low = 0, ep_line_high = 0;          // the lane's places in the two stores of store_c_lines (fp32: one piece; bf16: two pieces side by side)
    // One piece = the lane's eight consecutive n of MFMA tile row i and tile pair jp: scale, convert,
    // one 16-byte store (bf16) or two (fp32).
    auto piece_values = [&](auto I, auto JP, float (&v)[8]) __attribute__((always_inline)) {
        constexpr int i = decltype(I)::value, jp = decltype(JP)::value;
        const int cm = ep_m0 + wave_m * 128 + (PERM_A ? 8 * (r16 >> 2) + (r16 & 3) + 32 * (i >> 1) + 4 * (i & 1) : r16 + 16 * i);
        const int cn = ep_n0 + wave_n * 128 + 8 * g + 32 * jp;
        static_for<8>([&](auto E) {
            constexpr int e = decltype(E)::value;
            v[e] = acc_read<(i * 8 + 2 * jp + (e >> 2)) * 4 + (e & 3)>();
        });
        if constexpr (MODE == MODE_TENSOR) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] *= ep_ts;
        }
        if constexpr (MODE == MODE_ROWCOL) {
            // row/col scales were staged in LDS when the tile began
            const float* sc = (const float*)(smem + GEMM_LDS_BYTES + (ep_seq & 1) * ROWCOL_SCALE_BYTES);
            const float sa = sc[cm - ep_m0];
            const v4f lo = *(const v4f*)(sc + BM + (cn - ep_n0)), hi = *(const v4f*)(sc + BM + (cn - ep_n0) + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[e] *= lo[e] * sa;
                v[4 + e] *= hi[e] * sa;
            }
        }
    };
    // bf16, whole tiles: the pieces of tile pairs 2 jpp and 2 jpp + 1 of one MFMA tile row lie 64 bytes apart in every row;
    // the lanes of rows r and r + 8 exchange them (store_c_lines), and each of the two stores then writes eight whole
    // 128-byte lines instead of 64-byte halves of sixteen (a compute unit writes whole lines nearly twice as fast)
    auto store_line_pair = [&](auto I, auto JPP) __attribute__((always_inline)) {
        constexpr int i = decltype(I)::value, jpp = decltype(JPP)::value;
        float v0[8], v1[8];
        piece_values(I, std::integral_constant<int, 2 * jpp>{}, v0);
        piece_values(I, std::integral_constant<int, 2 * jpp + 1>{}, v1);
#ifdef A8W8_ABLATE_STORES
        asm volatile("" ::"v"(v0[0]), "v"(v0[7]), "v"(v1[0]), "v"(v1[7]));
        return;
#endif
        v4i w0, w1;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            w0[e] = bf16x2_bits(v0[2 * e], v0[2 * e + 1]);
            w1[e] = bf16x2_bits(v1[2 * e], v1[2 * e + 1]);
        }
        constexpr int row = PERM_A ? 32 * (i >> 1) + 4 * (i & 1) : 16 * i;
        store_c_lines<A8W8_WIDE_LINES_BY_LANE != 0>(ep_rs, w0, w1, r16 >= 8, ep_line_src_low, ep_line_src_high, ep_line_low + 128 * jpp, ep_line_high + 128 * jpp, (int)((uint32_t)row * (uint32_t)ep_row_bytes));
    };
    auto store_piece = [&](auto I, auto JP, bool checked) __attribute__((always_inline)) {
        constexpr int i = decltype(I)::value, jp = decltype(JP)::value;
        const int cm = ep_m0 + wave_m * 128 + (PERM_A ? 8 * (r16 >> 2) + (r16 & 3) + 32 * (i >> 1) + 4 * (i & 1) : r16 + 16 * i);
        const int cn = ep_n0 + wave_n * 128 + 8 * g + 32 * jp;
        char* c_base = (char*)p.c + (long long)ep_batch * p.c_batch * (CDT == C_BF16 ? 2 : 4);
        float v[8];
        piece_values(I, JP, v);
        if (!checked) {
            // a whole tile: through the tile's buffer descriptor
            constexpr int ES = CDT == C_BF16 ? 2 : 4;
            constexpr int row = PERM_A ? 32 * (i >> 1) + 4 * (i & 1) : 16 * i;
            const int voff = ep_lane_off + 32 * jp * ES, soff = (int)((uint32_t)row * (uint32_t)ep_row_bytes);
#ifdef A8W8_ABLATE_STORES
            asm volatile("" ::"v"(v[0]), "v"(v[7]), "s"(voff), "s"(soff));
            return;
#endif
            if constexpr (CDT == C_BF16) {
                v4i w;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = bf16x2_bits(v[2 * e], v[2 * e + 1]);
                store_c_16<A8W8_WIDE_WRITE_THROUGH != 0>(ep_rs, w, voff, soff);
            } else {
                (void)voff;
                store_c_lines<A8W8_WIDE_LINES_BY_LANE != 0>(ep_rs, __builtin_bit_cast(v4i, v4f{v[0], v[1], v[2], v[3]}), __builtin_bit_cast(v4i, v4f{v[4], v[5], v[6], v[7]}),
                              r16 >= 8, ep_line_src_low, ep_line_src_high, ep_line_low + 32 * jp * 4, ep_line_high + 32 * jp * 4, soff);
            }
            return;
        }
        if (cm >= p.m) return;
        const bool vec = ep_vec_ok && cn + 7 < p.n;
        if constexpr (CDT == C_BF16) {
            unsigned short* dst = (unsigned short*)c_base + (long long)cm * p.ldc + cn;
            if (vec) {
                v4i w;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = bf16x2_bits(v[2 * e], v[2 * e + 1]);
                A8W8_STORE_C((v4i*)dst, w);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (cn + e < p.n) dst[e] = bf16_bits(v[e]);
            }
        } else {
            float* dst = (float*)c_base + (long long)cm * p.ldc + cn;
            if (vec) {
                A8W8_STORE_C((v4f*)dst, (v4f{v[0], v[1], v[2], v[3]}));
                A8W8_STORE_C((v4f*)(dst + 4), (v4f{v[4], v[5], v[6], v[7]}));
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (cn + e < p.n) dst[e] = v[e];
            }
        }
    };
    // Piece g (0..7) of accumulator quadrant eq (0 aL x bL, 1 aL x bH, 2 aH x bL, 3 aH x bH), B-major (or
    // A-major when a_outer) like the quadrant's MFMAs.  Their inner index runs back and forth, so the
    // quadrant's last MFMA belongs to piece 4 (6 when a_outer), which is read ten (fourteen) MFMAs of
    // the next quadrant after it was issued; every other piece is further from its last MFMA.
    auto flush_piece = [&](auto EQ, auto GQ, auto AO) __attribute__((always_inline)) {
        constexpr int eq = decltype(EQ)::value, gq = decltype(GQ)::value;
        constexpr bool a_outer = decltype(AO)::value != 0;
        constexpr int i = (eq >> 1) * 4 + (a_outer ? (gq >> 1) : (gq & 3));
        constexpr int jp = (eq & 1) * 2 + (a_outer ? (gq & 1) : (gq >> 2));
        store_piece(std::integral_constant<int, i>{}, std::integral_constant<int, jp>{}, false);
    };
    // the whole tile with every bounds and alignment check, for tiles the pieces cannot serve
    auto store_tile_checked = [&]() __attribute__((always_inline)) {
        static_for<WIDE_T / 2>([&](auto JP) { static_for<WIDE_T>([&](auto I) { store_piece(I, JP, true); }); });
    };
    constexpr int STORES_PER_PIECE = CDT == C_BF16 ? 1 : 2;

    // ---------------------------------------------------------------- prologue
    const int my_items = (pp.items - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
    if (my_items == 0) return;
#ifdef A8W8_WIDE_STAGGER
    // measurement: workgroups start up to 7 * A8W8_WIDE_STAGGER * 64 clocks apart, so that their tiles do not all end at once
    for (int i = (int)((blockIdx.x * 0x9E37u >> 6) & 7u); i > 0; --i) __builtin_amdgcn_s_sleep(A8W8_WIDE_STAGGER);
#endif
    point_loads_at(ld_item);
    point_compute_at(cur_item);
    point_scales_at(sf_cur, cur_item);
    point_scales_at(sf_next, cur_item + (int)gridDim.x);
    issue_mx_batch(sf_cur, 0, 0);
    // Steps 0 and 1 in full.  Step 1's quarters go out in the order an odd step of the steady state issues
    // them (aL, bH, bL, aH): the hand-overs of the step that follows count on it.  Step 0's mid hand-over
    // waits for "all but the newest 16 loads"; by then aL and bL of step 2 have been issued behind step 1,
    // so what has landed is the first two quarters of step 1, and these must be the two that the second
    // half of step 0 reads: aL(1) and bH(1).  The end hand-over covers the other two.
#pragma unroll
    for (int st = 0; st < 2; ++st) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int qt = st == 0 ? q : (q == 0 ? 0 : 4 - q);
#pragma unroll
            for (int l = 0; l < 4; ++l) issue_one(st, qt, l);
        }
        advance_ld();
    }
    // vmcnt(16) lgkmcnt(0): step 0 and the first scale batch have landed; the 16 loads of step 1 may still be on their
    // way (the first step's hand-overs wait for them like for any other step's): 0.4 us less per launch
    __builtin_amdgcn_s_waitcnt(0x4070);
    A8W8_RAW_BARRIER();
    v8i fa[WIDE_T], fb[WIDE_T];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        fa[t] = read_frag_a(0, t);
        fb[t] = read_frag_b(0, t);
    }
    if constexpr (IS_MXT) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            sc_a[u] = *(const v2i*)(smem + rd_sfa + u * 1024);
            sc_b[u] = *(const v2i*)(smem + rd_sfb + u * 1024);
        }
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);
    A8W8_RAW_BARRIER();                              // the quarters just read may be overwritten from here on

    // ---------------------------------------------------------------- one quadrant
    // MFMAs of fa[IA..IA+3] x fb[JB..JB+3]; fragment set REF (0 aL, 1 aH, 2 bL, 3 bH) is re-read from
    // stage RS; quarter LQ of the step at the load position is issued into stage LS.  ZC: the tile's
    // first step, the MFMAs take zero instead of the accumulator.  EQ >= 0: the previous owner of
    // accumulator quadrant EQ is written out meanwhile, one piece per two MFMAs (EQA: that quadrant's
    // MFMAs ran A-major).
    bool have_prev = false;                         // a quadrant of the tile before is still to be written out
    auto quad = [&](auto IA, auto JB, auto REF, auto RS, auto LQ, auto LS, auto AOUTER, auto SPAR, auto SCREAD, auto ZC, auto EQ,
                    auto EQA) __attribute__((always_inline)) {
        constexpr bool a_outer = decltype(AOUTER)::value != 0;
        constexpr int sp = decltype(SPAR)::value;            // the step's parity: scale byte inside a pair
        constexpr bool SCR = decltype(SCREAD)::value != 0;   // this quadrant also fetches the next pair's scales
        constexpr bool zc = decltype(ZC)::value != 0;
        constexpr int eq = decltype(EQ)::value - 1;          // -1: nothing to write out
        constexpr bool eqa = decltype(EQA)::value != 0;
        constexpr int ia = decltype(IA)::value, jb = decltype(JB)::value, ref = decltype(REF)::value;
        constexpr int rs = decltype(RS)::value, lq = decltype(LQ)::value, ls = decltype(LS)::value;
        // The MFMAs are written as assembly statements: the accumulators stay in the accumulator
        // registers and are updated in place, and the statements keep their order, so the source
        // order below is the schedule: two MFMAs, one LDS read; a load after every fourth MFMA.
        v4i half[8];
        // 16 MPF slots: with two MFMAs per fragment pair, all first halves, then all second halves
        // (two MFMAs in a row on one accumulator would wait for each other)
        static_for<16 * MPF>([&](auto SS) {
            constexpr int sl = decltype(SS)::value;
            constexpr int hf = sl / 16, t = sl % 16;
            // the inner index runs back and forth, so that between any two consecutive MFMAs exactly one operand
            // changes (the matrix cores draw a little less power for it: 1-2% more sustained rate under the power limit)
            constexpr int inner = ((t >> 2) & 1) ? 3 - (t & 3) : (t & 3);
            constexpr int j = jb + (a_outer ? inner : (t >> 2)), i = ia + (a_outer ? (t >> 2) : inner);
            constexpr int lo = (i * 8 + j) * 4;
            constexpr bool z = zc && hf == 0;
            if constexpr (MODE == MODE_F4T) {
                const v4i bh = hf ? v4i{fb[j][4], fb[j][5], fb[j][6], fb[j][7]} : v4i{fb[j][0], fb[j][1], fb[j][2], fb[j][3]};
                const v4i ah = hf ? v4i{fa[i][4], fa[i][5], fa[i][6], fa[i][7]} : v4i{fa[i][0], fa[i][1], fa[i][2], fa[i][3]};
                mfma_acc_f4<lo, z, 2 * (j & 1) + hf, 2 * (i & 1) + hf>(bh, ah, sc_b[j >> 2][(j >> 1) & 1], sc_a[i >> 2][(i >> 1) & 1]);
            } else if constexpr (MODE == MODE_BF16) {
                // a 128-byte row is 64 bf16: both operands split K the same way, so the order of the
                // elements inside an instruction is immaterial
                const v4i bh = hf ? v4i{fb[j][4], fb[j][5], fb[j][6], fb[j][7]} : v4i{fb[j][0], fb[j][1], fb[j][2], fb[j][3]};
                const v4i ah = hf ? v4i{fa[i][4], fa[i][5], fa[i][6], fa[i][7]} : v4i{fa[i][0], fa[i][1], fa[i][2], fa[i][3]};
                mfma_acc_bf16<lo, z>(bh, ah);
            } else if constexpr (IS_MXT) {
#ifdef A8W8_ABLATE_UNSCALED_MFMA
                mfma_acc<lo, z>(fb[j], fa[i]);
#else
                mfma_acc_mx<lo, z, 2 * (j & 1) + sp, 2 * (i & 1) + sp>(fb[j], fa[i], sc_b[j >> 2][(j >> 1) & 1], sc_a[i >> 2][(i >> 1) & 1]);
#endif
            } else {
                mfma_acc<lo, z>(fb[j], fa[i]);
            }
            // The eight LDS reads of the quadrant go out behind its first eight MFMAs (A8W8_WIDE_READS_EARLY) rather than
            // one per two MFMAs to its end: the hand-over that follows every second quadrant waits for all of them, and a
            // read issued behind the last MFMA would leave the matrix cores idle for the whole of its latency.
            constexpr bool read_here = A8W8_WIDE_READS_EARLY ? (sl < 8 * MPF && sl % MPF == MPF - 1) : (sl % (2 * MPF) == 2 * MPF - 1);
            if constexpr (read_here) {
                constexpr int r = A8W8_WIDE_READS_EARLY ? sl / MPF : sl / (2 * MPF), f = (ref & 1) * 4 + (r >> 1), h = r & 1;     // half h of fragment f
                constexpr int par = f & 1;
                const int* base = ref < 2 ? rd_a : rd_b;
                constexpr int off = (f >> 1) * (32 * BK) + par * (ref < 2 ? A_PAR_BYTES : B_PAR_BYTES);
                half[r] = *(const v4i*)(smem + (rs * HALF_STAGE + off) + base[par ^ h]);
            }
#ifndef A8W8_ABLATE_OPERAND_LOADS
            if constexpr (sl % (4 * MPF) == 2 * MPF) issue_one(ls, lq, sl / (4 * MPF));
#endif
            if constexpr (IS_MXT && SCR && sl % (4 * MPF) == 0) {
                // the next pair's scales, four 8-byte reads spread over the quadrant
                constexpr int u = sl / (4 * MPF);
#ifdef A8W8_ABLATE_SCALE_READS
                const v2i v = u < 2 ? sc_a[u] : sc_b[u - 2];
#else
                const v2i v = *(const v2i*)(smem + sc_rd_off + (u < 2 ? rd_sfa : rd_sfb) + (u & 1) * 1024);
#endif
                if constexpr (u < 2) sc_a_next[u] = v;
                else sc_b_next[u - 2] = v;
            }
            if constexpr (eq >= 0 && sl % (2 * MPF) == 2 * MPF - 1) {
                using EQT = std::integral_constant<int, eq < 0 ? 0 : eq>;
                using GQT = std::integral_constant<int, sl / (2 * MPF)>;
                using AOT = std::integral_constant<int, eqa ? 1 : 0>;
                if constexpr (zc) {
                    if (have_prev) flush_piece(EQT{}, GQT{}, AOT{});
                } else {
                    flush_piece(EQT{}, GQT{}, AOT{});
                }
            }
        });
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const v4i lo = half[2 * t], hi = half[2 * t + 1];
            const v8i v = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            if constexpr (ref < 2) fa[(ref & 1) * 4 + t] = v;
            else fb[(ref & 1) * 4 + t] = v;
        }
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    using I4 = std::integral_constant<int, 4>;
    // Every LDS read issued so far is complete, and all memory operations but the newest N have
    // finished: N = the 16 loads of the last four quadrants plus the stores issued among them, so that
    // what has finished is exactly the two quarters the next two quadrants read.
    auto handover = [&](auto STORES) __attribute__((always_inline)) {
#if defined(A8W8_ABLATE_STORES) || defined(A8W8_ABLATE_STORE_INSTRUCTIONS)
        constexpr int want = 16;      // no stores are issued: the newest 16 operations are the loads
#else
        constexpr int want = 16 + decltype(STORES)::value * STORES_PER_PIECE;
#endif
        constexpr int n = want < 63 ? want : 63;             // a 6-bit counter; fewer is only stricter
        __builtin_amdgcn_s_waitcnt(((n & 15) | ((n >> 4) << 14)) | 0x0070);
        A8W8_RAW_BARRIER();
    };
    using S0 = std::integral_constant<int, 0>;
    using S8 = std::integral_constant<int, 8>;
    using S24 = std::integral_constant<int, 24>;
    using SALL = std::integral_constant<int, 32>;      // the whole tile's pieces (one wave's share)
    constexpr bool BURST = A8W8_WIDE_BURST != 0;

    // A K step.  FIRST: the tile's first step (even): accumulators start from zero, and the previous
    // tile's last quadrant is written out behind the first 16 MFMAs.  LAST: the tile's last step
    // (odd): each accumulator quadrant is written out behind the MFMAs of the quadrant after it.
    auto step = [&](auto parity, auto first, auto last) __attribute__((always_inline)) {
        constexpr int P = decltype(parity)::value;
        constexpr bool FIRST = decltype(first)::value != 0, LAST = decltype(last)::value != 0;
        static_assert(!(FIRST && P == 1) && !(LAST && P == 0), "tiles start on even steps and end on odd ones");
        // keeps the 32 LDS addresses of the loads from being computed once and parked in registers
        // (always wave * 1024, but tied to a value that changes with the step)
        wave_lds = wave * 1024 + (ld_ks >> 30);
        using SP = std::integral_constant<int, P>;
        using SN = std::integral_constant<int, P ^ 1>;
        using Z = std::integral_constant<int, FIRST ? 1 : 0>;
        if constexpr (P == 0) {
            // aL x bL | read bH of this step | load aL            (| write out aH x bH of the previous tile)
            quad(I0{}, I0{}, I3{}, SP{}, I0{}, SP{}, I0{}, SP{}, I0{}, Z{}, std::integral_constant<int, FIRST && !BURST ? 4 : 0>{}, I0{});
            // aL x bH | read aH of this step | load bL
            quad(I0{}, I4{}, I1{}, SP{}, I2{}, SP{}, I0{}, SP{}, I0{}, Z{}, I0{}, I0{});
            if constexpr (FIRST) {
                if (have_prev) handover(std::conditional_t<BURST, SALL, S24>{});
                else handover(S0{});
            } else {
                handover(S0{});
            }
            // aH x bH | read aL of the next step | load bH
            quad(I4{}, I4{}, I0{}, SN{}, I3{}, SP{}, I1{}, SP{}, I0{}, Z{}, I0{}, I0{});
            // aH x bL | read bH of the next step | load aH
            quad(I4{}, I0{}, I3{}, SN{}, I1{}, SP{}, I0{}, SP{}, std::integral_constant<int, PAIR_STEPS == 1 ? 1 : 0>{}, Z{}, I0{}, I0{});
            advance_ld();
            if constexpr (IS_MXT && PAIR_STEPS == 1) {
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    sc_a[u] = sc_a_next[u];
                    sc_b[u] = sc_b_next[u];
                }
            }
            if constexpr (FIRST) {
                if (have_prev) handover(std::conditional_t<BURST, SALL, S8>{});
                else handover(S0{});
            } else {
                handover(S0{});
            }
        } else {
            // aL x bH | read bL of this step | load aL
            quad(I0{}, I4{}, I2{}, SP{}, I0{}, SP{}, I0{}, SP{}, I0{}, I0{}, I0{}, I0{});
            // aL x bL | read aH of this step | load bH             (| write out aL x bH)
            quad(I0{}, I0{}, I1{}, SP{}, I3{}, SP{}, I0{}, SP{}, I0{}, I0{}, std::integral_constant<int, LAST ? 2 : 0>{}, I0{});
            if constexpr (LAST) handover(S8{});
            else handover(S0{});
            // aH x bL | read aL of the next step | load bL         (| write out aL x bL)
            quad(I4{}, I0{}, I0{}, SN{}, I2{}, SP{}, I1{}, SP{}, I0{}, I0{}, std::integral_constant<int, LAST ? 1 : 0>{}, I0{});
            // aH x bH | read bL of the next step | load aH         (| write out aH x bL, whose MFMAs ran A-major)
            quad(I4{}, I4{}, I2{}, SN{}, I1{}, SP{}, I0{}, SP{}, I1{}, I0{}, std::integral_constant<int, LAST ? 3 : 0>{}, I1{});
            advance_ld();
            if constexpr (IS_MXT) {
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    sc_a[u] = sc_a_next[u];
                    sc_b[u] = sc_b_next[u];
                }
            }
            if constexpr (LAST) handover(S24{});
            else handover(S0{});
        }
    };
    using F = std::integral_constant<int, 0>;
    using T = std::integral_constant<int, 1>;

    // The K loop of a tile is an even number of steps (checked by the host), so every tile starts on
    // an even step; loads and fragment reads run on across the tile boundary.
    for (int it = 0; it < my_items; ++it) {
        issue_rowcol_scales(cur_batch, m0, n0, tile_seq & 1);
        for (int ks = 0; ks < nk; ks += 2) {
            if constexpr (IS_MXT) {
                // at the first step of a batch of scale groups: fetch the next batch (of this tile or the
                // first of the next tile) into the other buffer; its first pair is read steps from here
                if (ks % BATCH_STEPS == 0) {
                    const int b1 = ks / BATCH_STEPS + 1;
#if defined(A8W8_ABLATE_SCALE_LOADS)
                    (void)b1;
#elif defined(A8W8_ABLATE_HOT_SCALES)
                    issue_mx_batch(sf_cur, 0, (cur_bbase + b1) & 1);
#else
                    if (b1 < batches_per_tile) issue_mx_batch(sf_cur, b1, (cur_bbase + b1) & 1);
                    else issue_mx_batch(sf_next, 0, (cur_bbase + batches_per_tile) & 1);
#endif
                }
            }
            // where the scales of the pair that starts at tile step `first` live (past the end: the next
            // tile's first pair)
            auto point_scale_read_at = [&](int first) __attribute__((always_inline)) {
                if constexpr (IS_MXT) {
                    const int q = first / PAIR_STEPS;          // pair; two pairs per scale group, GPB groups per batch
                    const bool same = first < nk;
                    const int buf = same ? (cur_bbase + (q >> 2)) & 1 : (cur_bbase + batches_per_tile) & 1;
                    sc_rd_off = buf * BATCH_BYTES + (same ? ((q >> 1) & 1) * MX_GROUP_BYTES + (q & 1) * 512 : 0);
                }
            };
            point_scale_read_at(PAIR_STEPS == 1 ? ks + 1 : ks + 2);
            if (ks == 0) step(F{}, T{}, F{});
            else step(F{}, F{}, F{});
            point_scale_read_at(ks + 2);
            if (ks + 2 == nk) {
                // from here on the accumulators are written out under this tile's coordinates
                ep_batch = cur_batch;
                ep_m0 = m0;
                ep_n0 = n0;
                ep_seq = tile_seq;
                if constexpr (MODE == MODE_TENSOR)
                    ep_ts = ((const float*)p.sfa + (long long)cur_batch * p.sfa_batch)[0] * ((const float*)p.sfb + (long long)cur_batch * p.sfb_batch)[0];
                const uintptr_t c_addr = (uintptr_t)p.c + (uintptr_t)((long long)cur_batch * p.c_batch * (CDT == C_BF16 ? 2 : 4));
                ep_vec_ok = (p.ldc & (CDT == C_BF16 ? 7 : 3)) == 0 && (c_addr & 15) == 0;
                // pieces are written without checks: only for whole tiles with aligned rows
                const bool fast = ep_vec_ok && m0 + BM <= p.m && n0 + BN <= p.n;
                {
                    constexpr int ES = CDT == C_BF16 ? 2 : 4;
                    ep_rs = make_rsrc((const char*)c_addr + ((long long)m0 * p.ldc + n0) * ES, (uint32_t)((BM - 1) * p.ldc + BN) * ES);
                    ep_row_bytes = p.ldc * ES;
                    auto row_of = [&](int r) __attribute__((always_inline)) { return PERM_A ? 8 * (r >> 2) + (r & 3) : r; };
                    // (unsigned arithmetic: with stride_c in the millions these byte offsets pass 2^31; the hardware takes them as unsigned)
                    ep_lane_off = (int)((uint32_t)(wave_m * 128 + row_of(r16)) * (uint32_t)ep_row_bytes + (uint32_t)((wave_n * 128 + 8 * g) * ES));
                    constexpr bool BL = A8W8_WIDE_LINES_BY_LANE != 0;
                    c_line_offsets<CDT == C_FP32 ? 16 : 64, BL>(lane, (int)((uint32_t)(wave_m * 128 + row_of(c_line_row<BL>(lane))) * (uint32_t)ep_row_bytes),
                                                                (int)((uint32_t)(wave_m * 128 + row_of(c_line_row<BL>(lane) + 8)) * (uint32_t)ep_row_bytes),
                                                                wave_n * 128 * ES, ep_line_low, ep_line_high);
                }
                if (fast && BURST) {
                    // The whole tile in one burst between its last step and the next tile's first: a store among the
                    // MFMAs makes its wave wait for a place in the memory pipeline, which the loads of the next steps
                    // share, and the K steps around a tile boundary then take three times as long as the others;
                    // written back to back the 32 stores of a wave cost less than they stretched those steps by.
                    // The next tile's first step lets them stay in flight (have_prev).
                    step(T{}, F{}, F{});
                    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // last MFMA -> first accumulator read
                    if constexpr (CDT == C_BF16 && A8W8_WIDE_LINE_PAIRS)
                        static_for<WIDE_T / 4>([&](auto JPP) { static_for<WIDE_T>([&](auto I) { store_line_pair(I, JPP); }); });
                    else
                        static_for<WIDE_T / 2>([&](auto JP) { static_for<WIDE_T>([&](auto I) { store_piece(I, JP, false); }); });
                    have_prev = true;
                } else if (fast) {
                    step(T{}, F{}, T{});
                    have_prev = true;
                } else {
                    step(T{}, F{}, F{});
                    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // last MFMA -> first accumulator read
                    store_tile_checked();
                    have_prev = false;
                }
            } else {
                step(T{}, F{}, F{});
            }
        }
        cur_bbase += batches_per_tile;
        ++tile_seq;
        cur_item += gridDim.x;
        point_compute_at(cur_item);
        sf_cur = sf_next;
        point_scales_at(sf_next, cur_item + (int)gridDim.x);
    }
    // the last tile's last quadrant (the compiler does not see the MFMAs: keep the required distance
    // between the last of them and the first read of an accumulator)
    if (have_prev && !BURST) {
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
        static_for<8>([&](auto GQ) { flush_piece(std::integral_constant<int, 3>{}, GQ, std::integral_constant<int, 0>{}); });
    }
    __builtin_amdgcn_s_waitcnt(0);   // no direct-to-LDS load may outlive the workgroup's LDS allocation
}

}  // namespace a8w8
