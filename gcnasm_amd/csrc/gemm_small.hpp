// Dense GEMM for problems too small to fill the chip with 256 x 256 tiles: 128 x 128 x 128 tile, 4 waves
// (2 along M x 2 along N), each wave owning a 64 x 64 block of C as 4 x 4 MFMA tiles of 16 x 16 x 128.
// A quarter of the work per workgroup means four times as many workgroups, and a problem of this size is
// bound by latency (first loads, the K loop's dependent steps, the C stores of one compute unit), not by the
// matrix cores.
//
// Data path as in the 256-tile kernels: 16-byte direct-to-LDS loads, 128-byte LDS rows whose 16-byte slots are
// XOR-swizzled with (row & 7), operand roles swapped so that a lane ends up with
// C[m = lane%16][n = 4*(lane/16) .. +3].  LDS stages of 32 KiB, four (loads three K steps ahead, one raw
// barrier per step) or two (see the kernel's template parameter).  Scales that change with the K step -- block
// scales, MX exponents -- ride in the same pipeline: each stage carries its step's scales, fetched by one extra
// direct-to-LDS load per wave, so that the loop's wait counts stay fixed and no global load has to be waited
// for inside a step.  Operands: FP8 E4M3, bf16 (byte rows of 2k columns), packed E2M1 (byte rows of k/2 columns).
#pragma once
#include "gemm_common.hpp"

namespace a8w8 {

constexpr int SM_BM = 128, SM_BN = 128;               // SM_BN: the widest tile; the kernel also takes 64 columns
constexpr int SM_THREADS = 256;
constexpr int small_stage_bytes(int bn) { return (SM_BM + bn) * BK; }   // 32768 for 128 columns, 24576 for 64
// Scale bytes per stage.  Block mode: 128 A-row scales, the B scale at +512 and +768.  Row-major MX: the step's
// four E8M0 bytes of 128 A rows, then of 128 B rows.  Tiled MX: 1 KiB per wave, whose first half is the 512-byte
// unit (64 rows x one pair of K steps) of the wave's row block.
// Row-major MX scales of packed E2M1 operands (MODE_F4): a 128-byte K step is 256 elements, eight E8M0 bytes per row:
// the rows' first dwords (128 A rows, then 128 B rows), then their second dwords.
constexpr int small_scale_bytes(int mode)
{
    return mode == MODE_MXT || mode == MODE_F4T ? 4096 : mode == MODE_F4 ? 2048 : (mode == MODE_BLOCK || mode == MODE_MX) ? 1024 : 0;
}
#ifndef A8W8_SMALL_PIPELINED
#define A8W8_SMALL_PIPELINED 1          // 0: loads in a block behind the barrier, fragments read in their own step (measurement)
#endif
#ifndef A8W8_SMALL_PIPELINED_TWO
#define A8W8_SMALL_PIPELINED_TWO 1      // the same switch for the two-stage variant
#endif
#ifndef A8W8_SMALL_LINES_BY_LANE
#define A8W8_SMALL_LINES_BY_LANE 1      // 0: whole tiles are stored from the MFMA layout as they are (measurement)
#endif
constexpr int SM_TM = 4;                               // MFMA tiles per wave along M (along N: a quarter of the tile's columns / 8)
constexpr int small_lds_bytes(int mode, int stages, int bn = SM_BN)
{
    return stages * (small_stage_bytes(bn) + small_scale_bytes(mode));
}

// p.tiles_m / p.tiles_n count 128 x 128 tiles here; grid = (tiles, 1, batch).  The launch bound asks for a
// 256-register budget: with 512 the compiler parks the block mode's partial tiles in accumulation registers
// and copies each value back before its multiply-add.
// SM_STAGES = 4: loads three K steps ahead, one barrier per step, one workgroup per compute unit (132-144 KiB of
// LDS) -- for grids of at most one workgroup per compute unit, where nothing else hides the load latency.
// SM_STAGES = 2: loads issued when a stage has been read, two barriers per step, two workgroups per compute unit
// that hide each other's waits -- for larger grids.
// BN_ = 64: tiles of 128 x 64 (a wave owns 64 x 32) for short, wide problems -- M of a few hundred rows over weights
// of many megabytes -- where 128 x 128 tiles would leave half of the compute units without a workgroup.  A workgroup
// alone on its compute unit streams its share of the weights through a long K loop: SM_STAGES = 6 there (five K
// steps of loads ahead, 144-154 KiB of LDS; 5 with tiled MX scales, whose 4 KiB per stage would not fit six; measured,
// five and six stages run alike, and so does a separate ring of ten stages for the weights).
template <int MODE, int CDT, int SM_STAGES, int BN_ = SM_BN>
__global__ void __launch_bounds__(SM_THREADS, 2) gemm_a8w8_tile128(GemmParams p)
{
    static_assert(SM_STAGES == 2 || SM_STAGES == 4 || SM_STAGES == 5 || SM_STAGES == 6, "two, four, five or six LDS stages");
    static_assert(BN_ == 128 || BN_ == 64, "tile width");
    constexpr int SM_BN = BN_;
    constexpr int SM_STAGE_BYTES = small_stage_bytes(SM_BN);
    constexpr int SM_TN = SM_BN / 32;                  // MFMA tiles per wave along N
    constexpr int B_LOADS = SM_BN / 32;                // 1 KiB chunks of B per wave and stage
    static_assert(MODE == MODE_TENSOR || MODE == MODE_ROWCOL || MODE == MODE_BLOCK || MODE == MODE_MX || MODE == MODE_MXT ||
                      MODE == MODE_BF16 || MODE == MODE_F4T || MODE == MODE_F4,
                  "fp32 scales, MX scales, bf16 operands (byte rows of 2k columns, no scales) or packed E2M1 operands (byte "
                  "rows of k/2 columns) with tiled MX scales");
    // tiled scales: of FP8 operands (a K step is 4 blocks of 32: one step of a pair) or of FP4 operands (8 blocks: a pair)
    constexpr bool TILED_SCALES = MODE == MODE_MXT || MODE == MODE_F4T;
    constexpr bool STEP_SCALES = MODE == MODE_BLOCK || MODE == MODE_MX || MODE == MODE_F4 || TILED_SCALES;      // scales that change with the K step
    constexpr bool IS_F4 = MODE == MODE_F4T || MODE == MODE_F4;      // packed E2M1 operands
    constexpr int SM_SCALE_BYTES = small_scale_bytes(MODE);
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = wave_uniform(tid >> 6);
    const int wave_m = wave >> 1, wave_n = wave & 1;
    const int batch = blockIdx.z;
    const int r16 = lane & 15, g = lane >> 4;

    int tile_m, tile_n;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * SM_BM, n0 = tile_n * SM_BN;
    const int nk = p.k / BK;

    const uint8_t* a_base = p.a + (long long)batch * p.a_batch;
    const uint8_t* b_base = p.b + (long long)batch * p.b_batch;
    const float* sfa_f = (const float*)p.sfa + (long long)batch * p.sfa_batch;
    const float* sfb_f = (const float*)p.sfb + (long long)batch * p.sfb_batch;
    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(a_base, (uint32_t)(p.m - 1) * p.lda + p.k);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(b_base, b_extent_bytes(p));

    // ---- global -> LDS.  A stage holds 16 A chunks then 16 (or 8) B chunks of 1 KiB (8 rows x 128 B); wave w
    // fills chunks w, w+4, .. of each matrix.  Lane i of a load lands on row i/8, slot i%8 of its
    // chunk and therefore fetches K-piece slot ^ (row & 7) = (i%8) ^ (i/8).
    const int ld_row = wave * 8 + (lane >> 3);
    const int ld_piece16 = ((lane & 7) ^ (lane >> 3)) * 16;
    int voff_a[4], voff_b[B_LOADS];
#pragma unroll
    for (int j = 0; j < 4; ++j) voff_a[j] = min(m0 + ld_row + 32 * j, p.m - 1) * p.lda + ld_piece16;
#pragma unroll
    for (int j = 0; j < B_LOADS; ++j) voff_b[j] = b_lane_offset(p, min(n0 + ld_row + 32 * j, p.n - 1), ld_piece16);
    // block mode: waves 0 and 1 fetch the step's 128 A-row scales (64 each), waves 2 and 3 the B scale
    // of the tile's 128 x 128 block (every lane the same dword: the stage's copy at +512 is the one read)
    constexpr int LOADS_PER_STAGE = 4 + B_LOADS + (MODE == MODE_F4 ? 2 : STEP_SCALES ? 1 : 0);
    __amdgpu_buffer_rsrc_t rsrc_sf = rsrc_a;
    int voff_sf = 0, sf_step_bytes = 0;
    if constexpr (MODE == MODE_BLOCK) {
        if (wave < 2) {
            rsrc_sf = make_rsrc(sfa_f, (uint32_t)((nk - 1) * p.stride_sfa + p.m) * 4u);
            voff_sf = min(m0 + wave * 64 + lane, p.m - 1) * 4;
            sf_step_bytes = p.stride_sfa * 4;
        } else {
            rsrc_sf = make_rsrc(sfb_f + (long long)(n0 >> 7) * p.stride_sfb, (uint32_t)nk * 4u);
            voff_sf = 0;
            sf_step_bytes = 4;
        }
    }
    // MX: waves 0 and 1 fetch the step's dword (four E8M0 bytes, one per 32 of K) of 64 A rows each, waves 2
    // and 3 those of 64 B rows each
    // (packed E2M1 operands: p.k counts bytes, a row has p.k / 16 scale bytes, eight per K step, fetched as two dwords)
    if constexpr (MODE == MODE_MX || MODE == MODE_F4) {
        const bool is_b = wave >= 2;
        const int rows = is_b ? p.n : p.m;
        const int stride = is_b ? p.stride_sfb : p.stride_sfa;
        const uint8_t* base = is_b ? (const uint8_t*)p.sfb + (long long)batch * p.sfb_batch
                                   : (const uint8_t*)p.sfa + (long long)batch * p.sfa_batch;
        rsrc_sf = make_rsrc(base, (uint32_t)(rows - 1) * stride + (uint32_t)(MODE == MODE_F4 ? p.k >> 4 : p.k >> 5));
        voff_sf = min((is_b ? n0 : m0) + (wave & 1) * 64 + lane, rows - 1) * stride;
        sf_step_bytes = MODE == MODE_F4 ? 8 : 4;
    }
    // tiled MX: wave w fetches the 512-byte unit of its 64-row block (waves 0, 1: the tile's A blocks, 2, 3: its B
    // blocks) for the step's pair of K steps with one 16-byte load; lanes 32-63 bring the next unit along, unused
    int mxt_nblk = 1, mxt_blk = 0;
    if constexpr (TILED_SCALES) {
        const bool is_b = wave >= 2;
        const int rows = is_b ? p.n : p.m;
        const uint8_t* base = is_b ? (const uint8_t*)p.sfb + (long long)batch * p.sfb_batch
                                   : (const uint8_t*)p.sfa + (long long)batch * p.sfa_batch;
        rsrc_sf = make_rsrc(base, (uint32_t)mx_tiled_bytes(rows, MODE == MODE_F4T ? 2 * p.k : p.k));      // k in elements
        voff_sf = lane * 16;
        mxt_nblk = (rows + 63) >> 6;
        // (a block past the last row: its rows are never stored; a 64-wide tile has one B block, wave 3 brings the next along unused)
        mxt_blk = min(((is_b ? n0 : m0) >> 6) + (wave & 1), mxt_nblk - 1);
    }
    auto issue_stage = [&](int stage, int kstep) __attribute__((always_inline)) {
        kstep = min(kstep, nk - 1);         // past the end: reload the last step into a stage nobody reads (fixed wait counts)
        A8W8_LDS char* s = (A8W8_LDS char*)smem + stage * SM_STAGE_BYTES + wave * 1024;
        const int koff = kstep * BK;
#pragma unroll
        for (int j = 0; j < 4; ++j) load_to_lds_16(rsrc_a, s + j * 4096, voff_a[j], koff);
#pragma unroll
        for (int j = 0; j < B_LOADS; ++j) load_to_lds_16(rsrc_b, s + SM_BM * BK + j * 4096, voff_b[j], kstep << p.b_kshift);
        if constexpr (TILED_SCALES) {
            A8W8_LDS char* sc = (A8W8_LDS char*)smem + SM_STAGES * SM_STAGE_BYTES + stage * SM_SCALE_BYTES + wave * 1024;
            // the pair of 128-element K steps this step belongs to (FP8: two byte steps) or is (FP4: 256 elements)
            const int pair = MODE == MODE_F4T ? kstep : kstep >> 1;
            load_to_lds_16(rsrc_sf, sc, voff_sf, ((((pair >> 1) * mxt_nblk + mxt_blk) * 2 + (pair & 1)) * 512));
        } else if constexpr (STEP_SCALES) {
            A8W8_LDS char* sc = (A8W8_LDS char*)smem + SM_STAGES * SM_STAGE_BYTES + stage * SM_SCALE_BYTES + wave * 256;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_sf, sc, 4, voff_sf, kstep * sf_step_bytes, 0, 0);
            if constexpr (MODE == MODE_F4) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_sf, sc + 1024, 4, voff_sf, kstep * sf_step_bytes + 4, 0, 0);
        }
    };

    // ---- LDS -> registers: a lane reads K-pieces g and g+4 of tile row r16; slot = piece ^ (row & 7), and
    // row & 7 = lane & 7 for every tile
    int rd_a[2], rd_b[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int slot = (g + 4 * h) ^ (lane & 7);
        rd_a[h] = (wave_m * 64 + r16) * BK + (slot << 4);
        rd_b[h] = SM_BM * BK + (wave_n * (SM_BN / 2) + r16) * BK + (slot << 4);
    }
    auto read_frag = [&](int stage, const int (&base)[2], int t) __attribute__((always_inline)) -> v8i {
        const char* s = smem + stage * SM_STAGE_BYTES + t * (16 * BK);
        const v4i lo = *(const v4i*)(s + base[0]);
        const v4i hi = *(const v4i*)(s + base[1]);
        return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    };

    // tiled MX: byte of (row 16 t + r16 of a 64-row block, 32-block g of the K step, step s of the pair) inside the
    // block's unit, without s (see mx_tiled_index); the same for A tiles and B tiles
    // (a 64-wide tile lies inside one 64-row block of B: wave column 1 owns the block's MFMA tiles 2 and 3)
    int mxt_off[4], mxt_off_b[SM_TN];
    const int mxt_unit_b = SM_BN == 128 ? (2 + wave_n) * 1024 : 2 * 1024;     // where the wave's B block lies in the stage's scale bytes
    if constexpr (TILED_SCALES) {
        auto unit_offset = [&](int t) __attribute__((always_inline)) {
            const int x = (2 * t + (r16 >> 3)) & 3, y = r16 & 3, par = (r16 >> 2) & 1;
            return ((4 * x + y) * 4 + g) * 8 + (t >> 1) * 4 + par * 2;
        };
#pragma unroll
        for (int t = 0; t < 4; ++t) mxt_off[t] = unit_offset(t);
#pragma unroll
        for (int t = 0; t < SM_TN; ++t) mxt_off_b[t] = unit_offset(SM_BN == 128 ? t : 2 * wave_n + t);
    }

    const int cm_base = m0 + wave_m * 64 + r16;          // + 16 * i
    const int cn_base = n0 + wave_n * (SM_BN / 2) + 4 * g;        // + 16 * j + e

    v4f acc[SM_TM][SM_TN];
#pragma unroll
    for (int i = 0; i < SM_TM; ++i)
#pragma unroll
        for (int j = 0; j < SM_TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    // Deep staging: the step's three instruction streams overlap inside the one wave of a SIMD.  The fragments (and
    // scales) of step ks + 1 are read from LDS while the MFMAs of step ks run (two register sets, the loop unrolled by
    // two), and the stage of step ks -- free as soon as everyone holds its fragments -- is refilled with step
    // ks + SM_STAGES by loads issued one at a time between those MFMAs.  Issued in a block behind the barrier, the loads
    // (which the compute unit's address path takes at 1 KiB per 7 ns), the LDS reads and the MFMAs follow one another:
    // 0.46 us per K step on 128 x 64 tiles where each of the three is 0.11-0.17 us.
    // Two stages (two workgroups per compute unit): there is no third stage to read ahead from, so a step reads all of its
    // fragments first, and behind a second barrier -- the stage is then free -- runs its MFMAs with the refill loads (step
    // ks + 2) between them; the other workgroup's MFMAs run beside this one's LDS reads.
    constexpr bool TWO = SM_STAGES == 2;
    constexpr bool PIPELINED = TWO ? A8W8_SMALL_PIPELINED_TWO != 0 : A8W8_SMALL_PIPELINED != 0;
    if constexpr (PIPELINED) {
        constexpr int HALVES = (IS_F4 || MODE == MODE_BF16) ? 2 : 1;      // MFMAs per pair of fragments
        constexpr int NFRAG = SM_TM + SM_TN, NSLOT = SM_TM * SM_TN * HALVES, NLOAD = LOADS_PER_STAGE;
        constexpr int LOAD_EVERY = NSLOT / NLOAD, READ_EVERY = NSLOT / NFRAG;
        constexpr int BLK_LAG = MODE == MODE_BLOCK ? 4 : 0;
        static_assert(LOAD_EVERY >= 1 && READ_EVERY >= 1 && (SM_STAGES - 1) * NLOAD < 64, "the wait count is a 6-bit field");
        v8i fr[TWO ? 1 : 2][NFRAG];       // A tiles, then B tiles
        int sc_a[TWO ? 1 : 2][SM_TM], sc_b[TWO ? 1 : 2][SM_TN];      // the step's scales: E8M0 bytes (MX modes), or the A-side factors as float bits (block)
        auto read_one = [&](int stage, int t) __attribute__((always_inline)) -> v8i {
            return t < SM_TM ? read_frag(stage, rd_a, t) : read_frag(stage, rd_b, t - SM_TM);
        };
        auto read_scales = [&](int stage, int ks, int (&sa)[SM_TM], int (&sb)[SM_TN]) __attribute__((always_inline)) {
            const char* sc = smem + SM_STAGES * SM_STAGE_BYTES + stage * SM_SCALE_BYTES;
            if constexpr (MODE == MODE_BLOCK) {
                const float* f = (const float*)sc;
                const float b = f[128];
#pragma unroll
                for (int t = 0; t < SM_TM; ++t) sa[t] = __builtin_bit_cast(int, f[wave_m * 64 + 16 * t + r16] * b);
            }
            if constexpr (MODE == MODE_MX) {
                // lane (r16, g) scales K [32g, 32g+32) of its row: byte g of the row's dword
                const unsigned* w = (const unsigned*)sc;
#pragma unroll
                for (int t = 0; t < SM_TM; ++t) sa[t] = (int)__builtin_amdgcn_ubfe(w[wave_m * 64 + 16 * t + r16], 8 * g, 8);
#pragma unroll
                for (int t = 0; t < SM_TN; ++t) sb[t] = (int)__builtin_amdgcn_ubfe(w[128 + wave_n * (SM_BN / 2) + 16 * t + r16], 8 * g, 8);
            }
            if constexpr (MODE == MODE_F4) {
                // lane (r16, g) scales 32-block g of each 128-element half of its row: byte g of the row's first and of
                // its second dword, put side by side as in the tiled layout (the half is chosen by op_sel)
                const unsigned* w = (const unsigned*)sc;
                auto two_bytes = [&](int row) __attribute__((always_inline)) {
                    return (int)(__builtin_amdgcn_ubfe(w[row], 8 * g, 8) | (__builtin_amdgcn_ubfe(w[256 + row], 8 * g, 8) << 8));
                };
#pragma unroll
                for (int t = 0; t < SM_TM; ++t) sa[t] = two_bytes(wave_m * 64 + 16 * t + r16);
#pragma unroll
                for (int t = 0; t < SM_TN; ++t) sb[t] = two_bytes(128 + wave_n * (SM_BN / 2) + 16 * t + r16);
            }
            if constexpr (MODE == MODE_F4T) {
                // both halves' bytes sit side by side: one 16-bit read, the half is chosen by op_sel
#pragma unroll
                for (int t = 0; t < SM_TM; ++t) sa[t] = *(const unsigned short*)(sc + wave_m * 1024 + mxt_off[t]);
#pragma unroll
                for (int t = 0; t < SM_TN; ++t) sb[t] = *(const unsigned short*)(sc + mxt_unit_b + mxt_off_b[t]);
            }
            if constexpr (MODE == MODE_MXT) {
                const uint8_t* u = (const uint8_t*)sc + (ks & 1);
#pragma unroll
                for (int t = 0; t < SM_TM; ++t) sa[t] = u[wave_m * 1024 + mxt_off[t]];
#pragma unroll
                for (int t = 0; t < SM_TN; ++t) sb[t] = u[mxt_unit_b + mxt_off_b[t]];
            }
        };
        // load n of a stage: four chunks of A, the chunks of B, then the step's scales
        auto load_one = [&](int stage, int kstep, int n) __attribute__((always_inline)) {
            A8W8_LDS char* s = (A8W8_LDS char*)smem + stage * SM_STAGE_BYTES + wave * 1024;
            if (n < 4) load_to_lds_16(rsrc_a, s + n * 4096, voff_a[n], kstep * BK);
            else if (n < 4 + B_LOADS) load_to_lds_16(rsrc_b, s + SM_BM * BK + (n - 4) * 4096, voff_b[n - 4], kstep << p.b_kshift);
            else if constexpr (TILED_SCALES) {
                A8W8_LDS char* sc = (A8W8_LDS char*)smem + SM_STAGES * SM_STAGE_BYTES + stage * SM_SCALE_BYTES + wave * 1024;
                const int pair = MODE == MODE_F4T ? kstep : kstep >> 1;
                load_to_lds_16(rsrc_sf, sc, voff_sf, ((((pair >> 1) * mxt_nblk + mxt_blk) * 2 + (pair & 1)) * 512));
            } else if constexpr (STEP_SCALES) {
                A8W8_LDS char* sc = (A8W8_LDS char*)smem + SM_STAGES * SM_STAGE_BYTES + stage * SM_SCALE_BYTES + wave * 256;
                if (n == 4 + B_LOADS) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_sf, sc, 4, voff_sf, kstep * sf_step_bytes, 0, 0);
                else __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_sf, sc + 1024, 4, voff_sf, kstep * sf_step_bytes + 4, 0, 0);
            }
        };
#pragma unroll
        for (int st = 0; st < SM_STAGES; ++st) issue_stage(st, st);
        if constexpr (!TWO) {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((SM_STAGES - 1) * NLOAD) : "memory");
            A8W8_RAW_BARRIER();
#pragma unroll
            for (int t = 0; t < NFRAG; ++t) fr[0][t] = read_one(0, t);
            read_scales(0, 0, sc_a[0], sc_b[0]);
        }
        // one K step: `have`, `sa`, `sb` hold its fragments and scales, the `next_` ones receive those of the step after it
        auto step = [&](int ks, int stage, v8i (&have)[NFRAG], int (&sa)[SM_TM], int (&sb)[SM_TN], v8i (&next)[NFRAG],
                        int (&next_sa)[SM_TM], int (&next_sb)[SM_TN]) __attribute__((always_inline)) {
            const int next_stage = stage + 1 == SM_STAGES ? 0 : stage + 1;
            if constexpr (TWO) {
                // this wave's loads of the step's stage have landed once only the other stage's are in flight; behind the
                // barrier everyone's have
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NLOAD) : "memory");
                A8W8_RAW_BARRIER();
#pragma unroll
                for (int t = 0; t < NFRAG; ++t) have[t] = read_one(stage, t);
                read_scales(stage, ks, sa, sb);
            }
            // this wave's loads of the next step's stage have landed once only the SM_STAGES - 2 younger stages are in
            // flight, and its reads of this step's fragments are complete: behind the barrier both hold for every wave
            if constexpr (!TWO) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((SM_STAGES - 2) * NLOAD) : "memory");
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            A8W8_RAW_BARRIER();
            const int kload = min(ks + SM_STAGES, nk - 1);      // past the end: the last step again, into a stage nobody reads
            v4f part[BLK_LAG + 1];
#pragma unroll
            for (int t = 0; t < NSLOT + BLK_LAG; ++t) {
                if (t < NSLOT) {
                    // fragments pairs column by column; two-MFMA pairs: first halves of the column's four tiles, then second
                    // halves (back-to-back MFMAs on one accumulator stall)
                    const int i = t % SM_TM, h = (t / SM_TM) % HALVES, j = t / (SM_TM * HALVES);
                    const v8i& fb = have[SM_TM + j];
                    const v8i& fa = have[i];
                    if constexpr (MODE == MODE_BLOCK) {
                        part[t % (BLK_LAG + 1)] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb, fa, v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                    } else if constexpr (IS_F4) {
                        // elements [0, 128) of the step sit in the fragments' first 16 bytes, [128, 256) in the second;
                        // op_sel picks the half's scale byte
                        if (h == 0)
                            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                                (v8i{fb[0], fb[1], fb[2], fb[3], 0, 0, 0, 0}), (v8i{fa[0], fa[1], fa[2], fa[3], 0, 0, 0, 0}), acc[i][j], 4, 4, 0,
                                sb[j], 0, sa[i]);
                        else
                            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                                (v8i{fb[4], fb[5], fb[6], fb[7], 0, 0, 0, 0}), (v8i{fa[4], fa[5], fa[6], fa[7], 0, 0, 0, 0}), acc[i][j], 4, 4, 1,
                                sb[j], 1, sa[i]);
                    } else if constexpr (MODE == MODE_MX || MODE == MODE_MXT) {
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb, fa, acc[i][j], 0, 0, 0, sb[j], 0, sa[i]);
                    } else if constexpr (MODE == MODE_BF16) {
                        // a 128-byte row is 64 bf16: the fragment's two 16-byte halves feed one 16x16x32 MFMA each
                        const v4i bh = {fb[4 * h], fb[4 * h + 1], fb[4 * h + 2], fb[4 * h + 3]};
                        const v4i ah = {fa[4 * h], fa[4 * h + 1], fa[4 * h + 2], fa[4 * h + 3]};
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, bh), __builtin_bit_cast(v8bf, ah), acc[i][j], 0, 0, 0);
                    } else {
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb, fa, acc[i][j], 0, 0, 0, 0, 0, 0);
                    }
                    if (t % LOAD_EVERY == 0 && t / LOAD_EVERY < NLOAD) load_one(stage, kload, t / LOAD_EVERY);
                    if constexpr (!TWO) {
                        if (t % READ_EVERY == 0 && t / READ_EVERY < NFRAG) next[t / READ_EVERY] = read_one(next_stage, t / READ_EVERY);
                        if (t == 0) read_scales(next_stage, ks + 1, next_sa, next_sb);
                    }
                }
                if constexpr (MODE == MODE_BLOCK) {
                    // acc += part * (sfa * sfb); the multiply-adds trail the MFMAs by BLK_LAG tiles so that they never
                    // wait on a matrix-core result that is still in flight
                    if (t >= BLK_LAG) {
                        const int u = t - BLK_LAG;
                        acc[u % SM_TM][u / SM_TM] += part[u % (BLK_LAG + 1)] * __builtin_bit_cast(float, sa[u % SM_TM]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            return next_stage;
        };
        int ks = 0, stage = 0;
        if constexpr (TWO) {
            for (; ks < nk; ++ks) stage = step(ks, stage, fr[0], sc_a[0], sc_b[0], fr[0], sc_a[0], sc_b[0]);
        } else {
            for (; ks + 1 < nk; ks += 2) {
                stage = step(ks, stage, fr[0], sc_a[0], sc_b[0], fr[1], sc_a[1], sc_b[1]);
                stage = step(ks + 1, stage, fr[1], sc_a[1], sc_b[1], fr[0], sc_a[0], sc_b[0]);
            }
            if (ks < nk) step(ks, stage, fr[0], sc_a[0], sc_b[0], fr[1], sc_a[1], sc_b[1]);
        }
    } else {
    issue_stage(0, 0);
    issue_stage(1, 1);
    if constexpr (SM_STAGES > 2) {
#pragma unroll
        for (int st = 2; st < SM_STAGES - 1; ++st) issue_stage(st, st);
    }
    // stages in flight behind the one being read: one of two, else all but the one being refilled
    constexpr int YOUNGER = SM_STAGES == 2 ? 1 : SM_STAGES - 2;
    static_assert(YOUNGER * LOADS_PER_STAGE < 64, "the wait count is a 6-bit field");

    int cur = 0, refill = SM_STAGES - 1;      // the stage of step ks, the stage of step ks - 1 (refilled with step ks + SM_STAGES - 1)
    for (int ks = 0; ks < nk; ++ks) {
        // this wave's loads of stage `cur` have landed once only the younger stages are in flight
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(YOUNGER * LOADS_PER_STAGE) : "memory");
        A8W8_RAW_BARRIER();                 // ... everyone's have; and (more than two stages) everyone is done reading the stage of step ks-1
        if constexpr (SM_STAGES > 2) issue_stage(refill, ks + SM_STAGES - 1);

        v8i fa[SM_TM], fb[2];
#pragma unroll
        for (int t = 0; t < SM_TM; ++t) fa[t] = read_frag(cur, rd_a, t);
        fb[0] = read_frag(cur, rd_b, 0);
        if constexpr (MODE == MODE_BLOCK) {
            const float* sc = (const float*)(smem + SM_STAGES * SM_STAGE_BYTES + cur * SM_SCALE_BYTES);
            const float sb = sc[128];
            float blk_s[SM_TM];
#pragma unroll
            for (int t = 0; t < SM_TM; ++t) blk_s[t] = sc[wave_m * 64 + 16 * t + r16] * sb;
            // acc += part * (sfa * sfb); the multiply-adds trail the MFMAs by BLK_LAG tiles so that they never
            // wait on a matrix-core result that is still in flight
            constexpr int BLK_LAG = 4;
            v4f part[BLK_LAG + 1];
#pragma unroll
            for (int t = 0; t < SM_TM * SM_TN + BLK_LAG; ++t) {
                if (t < SM_TM * SM_TN) {
                    const int j = t / SM_TM, i = t % SM_TM;
                    if (i == 0 && j + 1 < SM_TN) fb[(j + 1) & 1] = read_frag(cur, rd_b, j + 1);
                    part[t % (BLK_LAG + 1)] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                        fb[j & 1], fa[i], v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);   // keep the lag: the scheduler would pull the FMAs up
                if (t >= BLK_LAG) {
                    const int u = t - BLK_LAG;
                    acc[u % SM_TM][u / SM_TM] += part[u % (BLK_LAG + 1)] * blk_s[u % SM_TM];
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            int mx_sa[SM_TM], mx_sb[SM_TN];
            if constexpr (MODE == MODE_MX) {
                // lane (r16, g) scales K [32g, 32g+32) of its row: byte g of the row's dword
                const unsigned* sc = (const unsigned*)(smem + SM_STAGES * SM_STAGE_BYTES + cur * SM_SCALE_BYTES);
#pragma unroll
                for (int t = 0; t < SM_TM; ++t) mx_sa[t] = (int)__builtin_amdgcn_ubfe(sc[wave_m * 64 + 16 * t + r16], 8 * g, 8);
#pragma unroll
                for (int t = 0; t < SM_TN; ++t) mx_sb[t] = (int)__builtin_amdgcn_ubfe(sc[128 + wave_n * (SM_BN / 2) + 16 * t + r16], 8 * g, 8);
            }
            if constexpr (MODE == MODE_F4) {
                // lane (r16, g) scales 32-block g of each 128-element half of its row: byte g of the row's first and of
                // its second dword, put side by side as in the tiled layout (the half is chosen by op_sel)
                const unsigned* sc = (const unsigned*)(smem + SM_STAGES * SM_STAGE_BYTES + cur * SM_SCALE_BYTES);
                auto two_bytes = [&](int row) __attribute__((always_inline)) {
                    return (int)(__builtin_amdgcn_ubfe(sc[row], 8 * g, 8) | (__builtin_amdgcn_ubfe(sc[256 + row], 8 * g, 8) << 8));
                };
#pragma unroll
                for (int t = 0; t < SM_TM; ++t) mx_sa[t] = two_bytes(wave_m * 64 + 16 * t + r16);
#pragma unroll
                for (int t = 0; t < SM_TN; ++t) mx_sb[t] = two_bytes(128 + wave_n * (SM_BN / 2) + 16 * t + r16);
            }
            if constexpr (MODE == MODE_F4T) {
                // both halves' bytes sit side by side: one 16-bit read, the half is chosen by op_sel
                const char* sc = smem + SM_STAGES * SM_STAGE_BYTES + cur * SM_SCALE_BYTES;
#pragma unroll
                for (int t = 0; t < SM_TM; ++t) mx_sa[t] = *(const unsigned short*)(sc + wave_m * 1024 + mxt_off[t]);
#pragma unroll
                for (int t = 0; t < SM_TN; ++t) mx_sb[t] = *(const unsigned short*)(sc + mxt_unit_b + mxt_off_b[t]);
            }
            if constexpr (MODE == MODE_MXT) {
                const uint8_t* sc = (const uint8_t*)(smem + SM_STAGES * SM_STAGE_BYTES + cur * SM_SCALE_BYTES) + (ks & 1);
#pragma unroll
                for (int t = 0; t < SM_TM; ++t) mx_sa[t] = sc[wave_m * 1024 + mxt_off[t]];
#pragma unroll
                for (int t = 0; t < SM_TN; ++t) mx_sb[t] = sc[mxt_unit_b + mxt_off_b[t]];
            }
#pragma unroll
            for (int j = 0; j < SM_TN; ++j) {
                if (j + 1 < SM_TN) fb[(j + 1) & 1] = read_frag(cur, rd_b, j + 1);
                if constexpr (IS_F4) {
                    // two FP4 MFMAs per fragment pair: elements [0, 128) of the step sit in the fragments' first 16
                    // bytes, [128, 256) in the second; op_sel picks the half's scale byte
#pragma unroll
                    for (int i = 0; i < SM_TM; ++i) {
                        const v8i& fbj = fb[j & 1];
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                            (v8i{fbj[0], fbj[1], fbj[2], fbj[3], 0, 0, 0, 0}), (v8i{fa[i][0], fa[i][1], fa[i][2], fa[i][3], 0, 0, 0, 0}),
                            acc[i][j], 4, 4, 0, mx_sb[j], 0, mx_sa[i]);
                    }
#pragma unroll
                    for (int i = 0; i < SM_TM; ++i) {
                        const v8i& fbj = fb[j & 1];
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                            (v8i{fbj[4], fbj[5], fbj[6], fbj[7], 0, 0, 0, 0}), (v8i{fa[i][4], fa[i][5], fa[i][6], fa[i][7], 0, 0, 0, 0}),
                            acc[i][j], 4, 4, 1, mx_sb[j], 1, mx_sa[i]);
                    }
                } else if constexpr (MODE == MODE_MX || MODE == MODE_MXT) {
#pragma unroll
                    for (int i = 0; i < SM_TM; ++i)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[j & 1], fa[i], acc[i][j], 0, 0, 0, mx_sb[j], 0,
                                                                                     mx_sa[i]);
                } else if constexpr (MODE == MODE_BF16) {
                    // a 128-byte row is 64 bf16: the fragment's two 16-byte halves feed one 16x16x32 MFMA each (both
                    // operands split K the same way); first halves for all four tiles, then second halves:
                    // back-to-back MFMAs on one accumulator stall
#pragma unroll
                    for (int h = 0; h < 2; ++h)
#pragma unroll
                        for (int i = 0; i < SM_TM; ++i) {
                            const v8i& fbj = fb[j & 1];
                            const v4i bh = {fbj[4 * h], fbj[4 * h + 1], fbj[4 * h + 2], fbj[4 * h + 3]};
                            const v4i ah = {fa[i][4 * h], fa[i][4 * h + 1], fa[i][4 * h + 2], fa[i][4 * h + 3]};
                            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, bh), __builtin_bit_cast(v8bf, ah),
                                                                                acc[i][j], 0, 0, 0);
                        }
                } else {
#pragma unroll
                    for (int i = 0; i < SM_TM; ++i)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[j & 1], fa[i], acc[i][j], 0, 0, 0, 0, 0, 0);
                }
            }
        }
        if constexpr (SM_STAGES == 2) {
            // everyone is done reading stage `cur`: refill it with the step after next (the next step's wait lets
            // exactly these loads stay in flight)
            A8W8_RAW_BARRIER();
            issue_stage(cur, ks + 2);
        }
        refill = cur;
        cur = cur + 1 == SM_STAGES ? 0 : cur + 1;
    }
    }

    // ---- epilogue: dequantise in fp32, convert, store
    float sa[SM_TM];
    float ts = 1.f;
    if constexpr (MODE == MODE_TENSOR) ts = sfa_f[0] * sfb_f[0];
    if constexpr (MODE == MODE_ROWCOL) {
#pragma unroll
        for (int i = 0; i < SM_TM; ++i) sa[i] = sfa_f[min(cm_base + 16 * i, p.m - 1)];
    }
    char* c_base = (char*)p.c + (long long)batch * p.c_batch * (CDT == C_BF16 ? 2 : 4);
    const bool vec_ok = (CDT == C_BF16) ? ((p.ldc & 3) == 0 && (((uintptr_t)c_base) & 7) == 0)
                                        : ((p.ldc & 3) == 0 && (((uintptr_t)c_base) & 15) == 0);
    const bool whole = vec_ok && m0 + SM_BM <= p.m && n0 + SM_BN <= p.n;
#if A8W8_SMALL_LINES_BY_LANE
    // A tile inside the matrix leaves through LDS, 16 rows of the wave's 64 at a time: the MFMA layout's stores have
    // neighbouring lanes in different rows (16 rows x 16 bytes per 16 lanes), which occupies the memory pipeline 2.7 times as long as
    // stores whose consecutive lanes write consecutive 16 bytes of a row.  A problem of few tiles ends with every workgroup's stores
    // and nothing to hide them behind.  The wave writes the 16 x (16 SM_TN) values into its own 4.25 KiB of LDS (rows padded
    // by 16 bytes against bank conflicts), reads them back along the rows and stores 16 bytes per lane; a wave's LDS
    // operations complete in order, so neither step needs a barrier.  Every direct-to-LDS load has landed by then (the
    // loop's last loads re-fill stages nobody reads).
    if (whole && (CDT == C_FP32 ? (p.ldc & 3) == 0 : (p.ldc & 7) == 0) && (((uintptr_t)c_base) & 15) == 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        constexpr int ES = CDT == C_BF16 ? 2 : 4;
        constexpr int ROW_BYTES = SM_TN * 16 * ES;                 // the wave's columns of one row
        constexpr int ROW_PITCH = ROW_BYTES + 16;
        constexpr int LANES_PER_ROW = ROW_BYTES / 16, ROWS_PER_STORE = 64 / LANES_PER_ROW, STORES = 16 / ROWS_PER_STORE;
        char* mine = smem + wave * (16 * (SM_BN / 2 * 4 + 16));
        const int wr = r16 * ROW_PITCH + 4 * g * ES;              // + 16 j ES: the lane's four values of MFMA tile j
        const int rd = (lane / LANES_PER_ROW) * ROW_PITCH + (lane % LANES_PER_ROW) * 16;      // + ROWS_PER_STORE rows per store
        char* c_wave = c_base + ((long long)(m0 + wave_m * 64) * p.ldc + n0 + wave_n * (SM_BN / 2)) * ES;
        const long long row_bytes = (long long)p.ldc * ES;
        float sb_all[SM_TN][4];
        if constexpr (MODE == MODE_ROWCOL) {
#pragma unroll
            for (int j = 0; j < SM_TN; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) sb_all[j][e] = sfb_f[cn_base + 16 * j + e];
        }
#pragma unroll
        for (int i = 0; i < SM_TM; ++i) {
#pragma unroll
            for (int j = 0; j < SM_TN; ++j) {
                v4f v = acc[i][j];
                if constexpr (MODE == MODE_TENSOR) v *= ts;
                if constexpr (MODE == MODE_ROWCOL) v *= v4f{sb_all[j][0], sb_all[j][1], sb_all[j][2], sb_all[j][3]} * sa[i];
                if constexpr (CDT == C_BF16) *(v2i*)(mine + wr + 16 * j * ES) = v2i{bf16x2_bits(v.x, v.y), bf16x2_bits(v.z, v.w)};
                else *(v4f*)(mine + wr + 16 * j * ES) = v;
            }
#pragma unroll
            for (int st = 0; st < STORES; ++st) {
                const v4i w = *(const v4i*)(mine + rd + st * ROWS_PER_STORE * ROW_PITCH);
                const int row = 16 * i + st * ROWS_PER_STORE + lane / LANES_PER_ROW;
                A8W8_STORE_C((v4i*)(c_wave + row * row_bytes + (lane % LANES_PER_ROW) * 16), w);
            }
        }
        return;
    }
#endif
#pragma unroll
    for (int j = 0; j < SM_TN; ++j) {
        const int cn = cn_base + 16 * j;
        v4f sb = v4f{1.f, 1.f, 1.f, 1.f};
        if constexpr (MODE == MODE_ROWCOL) {
#pragma unroll
            for (int e = 0; e < 4; ++e) sb[e] = sfb_f[min(cn + e, p.n - 1)];
        }
#pragma unroll
        for (int i = 0; i < SM_TM; ++i) {
            const int cm = cm_base + 16 * i;
            v4f v = acc[i][j];
            if constexpr (MODE == MODE_TENSOR) v *= ts;
            if constexpr (MODE == MODE_ROWCOL) v *= sb * sa[i];
            if (whole) {        // inside the matrix, aligned rows: no per-lane checks
                if constexpr (CDT == C_BF16)
                    A8W8_STORE_C((v2i*)((unsigned short*)c_base + (long long)cm * p.ldc + cn), (v2i{bf16x2_bits(v.x, v.y), bf16x2_bits(v.z, v.w)}));
                else
                    A8W8_STORE_C((v4f*)((float*)c_base + (long long)cm * p.ldc + cn), v);
                continue;
            }
            if (cm >= p.m) continue;
            if constexpr (CDT == C_BF16) {
                unsigned short* dst = (unsigned short*)c_base + (long long)cm * p.ldc + cn;
                if (vec_ok && cn + 3 < p.n) {
                    A8W8_STORE_C((v2i*)dst, (v2i{bf16x2_bits(v.x, v.y), bf16x2_bits(v.z, v.w)}));
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
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no direct-to-LDS load may outlive the workgroup's LDS allocation
}

}  // namespace a8w8
