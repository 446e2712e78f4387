// Skinny-M ("flat") A8W8 GEMM over pre-shuffled weights for gfx950.
//
// B arrives as Bshuf[n/16][k/64][4][16][16 B]: one 1 KiB block per (16 rows of B, 64 K),
// ordered so that a 64-lane load of 16 bytes per lane is one contiguous 1 KiB read and lane
// (kq = lane/16, r = lane%16) receives K bytes [16kq, 16kq+16) of row r -- half of a
// 16 x 16 x 128 MFMA operand.  Two consecutive K blocks make one MFMA; the activation
// fragment is gathered with the same K order, so for up to 16 activation rows no data moves through LDS.
//
// The kernel is bound by HBM: B is read exactly once with non-temporal 16-byte loads.
// A workgroup is 8 waves that split K eight ways for the same NT weight tiles and up to four groups of 16
// activation rows (all waves stream B concurrently, the activation fragment of a K block is shared by the NT
// tiles); the partial 16 x 16 accumulators are reduced through LDS and the dequantisation scales are applied in
// fp32 before the store.
//
// The same kernel runs MXFP4: A and B hold packed E2M1 (two elements per byte), B pre-shuffled as the byte matrix
// [n][k/2] with the same 1 KiB blocks -- a block is 16 rows x 64 bytes = 16 rows x 128 elements, exactly one
// operand of the FP4 form of the 16 x 16 x 128 MFMA (lane (kq, r) supplies elements [32 kq, 32 kq + 32) of row r,
// one 32-element scale block).  E8M0 scales of both operands come in the tiled layout of the dense kernels
// (mx_tiled_index): the two bytes of (row, 32-block) for the two 128-element blocks of a pair sit side by side, so
// a lane fetches one 16-bit word per tile and pair of blocks and op_sel picks the block's byte.  p.k and p.lda
// then count bytes (half the element counts).
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
    if (m_tiles == 1) {      // the common case without its divisions: every cycle before the first load is a cycle of idle memory
        m_tile = 0;
        n_group = bid;
    } else if ((n_groups & 7) == 0) {
        const int rest = bid >> 3;
        m_tile = rest % m_tiles;
        n_group = (rest / m_tiles) * 8 + (bid & 7);
    } else {
        m_tile = bid % m_tiles;
        n_group = bid / m_tiles;
    }
}

// 16 bytes per lane through a buffer descriptor: lane offset in a register, the rest of the address scalar.
A8W8_DEV v4i ld16(__amdgpu_buffer_rsrc_t rs, uint32_t voffset, int soffset)
{
    return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rs, voffset, soffset, 0));
}
// The same marked non-temporal (streamed once: no reason to keep it in cache).
A8W8_DEV v4i ld16_nt(__amdgpu_buffer_rsrc_t rs, uint32_t voffset, int soffset)
{
    return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rs, voffset, soffset, 2));
}

// Activation rows of one pair of K blocks, staged per wave for MT > 1: 8 pieces of 16 bytes per row (piece c of
// a 128-byte line), piece-major with a stride of 18 slots so that both the row-wise writes and the piece-wise reads
// touch every LDS bank once.
constexpr int FLAT_STAGE_SLOTS = 8 * 18;

// Scaled FP8 MFMA whose two E8M0 scales are bytes `byte_b` / `byte_a` (0 .. 3, constants once the caller's loops are
// unrolled) of the registers sb / sa.
template <int OB, int OA>
A8W8_DEV v4f mfma_mx_sel(v8i b, v8i a, v4f c, int sb, int sa)
{
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b, a, c, 0, 0, OB, sb, OA, sa);
}
A8W8_DEV v4f mfma_mx_bytes(v8i b, v8i a, v4f c, int byte_b, int sb, int byte_a, int sa)
{
    switch (byte_b * 4 + byte_a) {
#define A8W8_MX_CASE(B, A) case B * 4 + A: return mfma_mx_sel<B, A>(b, a, c, sb, sa);
        A8W8_MX_CASE(0, 0) A8W8_MX_CASE(0, 1) A8W8_MX_CASE(0, 2) A8W8_MX_CASE(0, 3)
        A8W8_MX_CASE(1, 0) A8W8_MX_CASE(1, 1) A8W8_MX_CASE(1, 2) A8W8_MX_CASE(1, 3)
        A8W8_MX_CASE(2, 0) A8W8_MX_CASE(2, 1) A8W8_MX_CASE(2, 2) A8W8_MX_CASE(2, 3)
        A8W8_MX_CASE(3, 0) A8W8_MX_CASE(3, 1) A8W8_MX_CASE(3, 2) A8W8_MX_CASE(3, 3)
#undef A8W8_MX_CASE
    }
    return c;
}

// MT groups of 16 activation rows per workgroup share one pass over the weights.  With MT = 1 a lane gathers its
// MFMA fragment straight from memory (16 bytes of one row per lane: 16 cache lines per quarter wave, affordable
// once per pair of K blocks).  With MT > 1 that gather would cost more than the weight stream, so the wave reads
// the rows the coalesced way (eight lanes per 128-byte line) and turns them into fragments through a private
// piece of LDS; nothing is shared between waves, so the K loop still has no barrier.
//
// BROW: the weights are row-major ([n][ldb], not pre-shuffled).  Their 16-row tiles then take the road of the
// activation rows of MT > 1: read the coalesced way, one register set in flight, through the wave's LDS into fragments.
template <int NT, int MT, int CDT, int MODE, bool BROW = false>
__global__ void __launch_bounds__(FLAT_THREADS) flatmm_a8w8(GemmParams p)
{
    // the NT * MT output tiles are finished in rounds of up to eight, wave w taking tile 8 * round + w of the round
    constexpr int TILES = NT * MT;
    constexpr int ROUNDS = (TILES + FLAT_WAVES - 1) / FLAT_WAVES;
    constexpr int RED_SLOTS = FLAT_WAVES * (TILES < FLAT_WAVES ? TILES : FLAT_WAVES) * 64;
    constexpr int A_GROUPS = MT > 1 ? MT : 0;                 // staged row groups of A, then NT of row-major B
    constexpr int STAGED = A_GROUPS + (BROW ? NT : 0);
    constexpr int STAGE_SLOTS = FLAT_WAVES * STAGED * FLAT_STAGE_SLOTS;
    __shared__ v4i smem[RED_SLOTS > STAGE_SLOTS ? RED_SLOTS : STAGE_SLOTS];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = wave_uniform(tid >> 6);
    const int batch = blockIdx.z;
    const int r16 = lane & 15, kq = lane >> 4;

    // What the epilogue needs of the arguments is read now and kept in registers: left to itself the compiler fetches
    // it from the argument block after the K loop, a scalar load that misses its cache at the one point where the
    // whole workgroup waits for it.
    int ldc = p.ldc;
    long long c_batch_off = (long long)batch * p.c_batch;
    asm volatile("" : "+s"(ldc), "+s"(c_batch_off));
    const int n_tiles = p.n >> 4;
    const int k_tiles = p.k >> 6;
    int n_group, m_tile_;
    flat_work_of_block(blockIdx.x, (n_tiles + NT - 1) / NT, (p.m + 16 * MT - 1) / (16 * MT), n_group, m_tile_);
    const int nt0 = n_group * NT;
    const int m0 = m_tile_ * (16 * MT);

    // Output tile c = g * NT + t is weight tile t of row group g; a finishing lane holds
    // C[m = r16 of the group][n = tile*16 + 4*kq .. +3].  Its scales are fetched now, so that the tail of the kernel
    // is only reduce + store.
    int cm[ROUNDS], cn[ROUNDS];
    bool finisher[ROUNDS];
    float sa[ROUNDS];
    v4f sb[ROUNDS];
    auto fetch_scales = [&](int r) {
        const int c = r * FLAT_WAVES + wave;
        const int fin_t = c % NT, fin_g = c / NT;
        cm[r] = m0 + fin_g * 16 + r16;
        cn[r] = (nt0 + fin_t) * 16 + 4 * kq;
        finisher[r] = c < TILES && cm[r] < p.m && nt0 + fin_t < n_tiles;
        sa[r] = 1.f;
        sb[r] = v4f{1.f, 1.f, 1.f, 1.f};
        if (finisher[r]) {
            const float* sfa = (const float*)p.sfa + (long long)batch * p.sfa_batch;
            const float* sfb = (const float*)p.sfb + (long long)batch * p.sfb_batch;
            if constexpr (MODE == MODE_BF16 || MODE == MODE_MXT || MODE == MODE_F4T || MODE == MODE_BLOCK) {
                // bf16 operands carry no scales; MX scales go into the MFMAs, block scales into the K loop
            } else if constexpr (MODE == MODE_TENSOR) {
                sa[r] = sfa[0] * sfb[0];
            } else {
                sa[r] = sfa[cm[r]];
                sb[r] = v4f{sfb[cn[r]], sfb[cn[r] + 1], sfb[cn[r] + 2], sfb[cn[r] + 3]};
            }
        }
    };
    // (fetched once the first weight loads are under way; with more rounds than one the registers are worth more than
    // the head start and the fetch waits until the K loop is over)

    // MT = 1: lane (r16, kq) reads bytes [16 kq, 16 kq + 16) of row r16 in each K block.
    // MT > 1: lane (row = lane / 4, c = lane % 4) reads bytes [32 c, 32 c + 32) of the pair's 128-byte line.
    // Staged rows (A for MT > 1, row-major B): lane (row = lane / 8, piece = lane % 8) reads 16-byte piece `piece` of
    // the pair's 128-byte line of row `row`, and of row + 8 with a second load: eight whole lines per instruction.
    const int ld_row = lane >> 3;
    const int ld_piece = lane & 7;
    // addresses are a wave-uniform base plus a 32-bit lane offset (operand extents are below 2 GiB): one register
    // per row group and weight tile instead of a 64-bit pointer each
    // (buffer loads: descriptor + 32-bit lane offset + scalar offset, so no load needs a 64-bit address in registers)
    const auto rs_a = make_rsrc(p.a + (long long)batch * p.a_batch, (uint32_t)(p.m - 1) * (uint32_t)p.lda + (uint32_t)p.k);
    uint32_t a_off[MT];
#pragma unroll
    for (int g = 0; g < MT; ++g)
        a_off[g] = MT == 1 ? (uint32_t)min(m0 + r16, p.m - 1) * (uint32_t)p.lda + kq * 16
                           // rows past m lie beyond the descriptor's extent and read as zero: no clamp
                           : (uint32_t)(m0 + g * 16 + ld_row) * (uint32_t)p.lda + ld_piece * 16;
    v4i* stage = smem + wave * (STAGED * FLAT_STAGE_SLOTS);
    const uint32_t kill_second = ld_piece >= 4 ? 0x80000000u : 0u;
    const int st_write = ld_piece * 18 + ld_row;         // row + 8 is 8 slots on
    const int st_read = kq * 18 + r16;                   // piece kq, the second K block's is 4 * 18 slots on

    const auto rs_b = make_rsrc(p.b + (long long)batch * p.b_batch, BROW ? (uint32_t)(p.n - 1) * (uint32_t)p.ldb + (uint32_t)p.k
                                                                         : (uint32_t)p.n * (uint32_t)p.k);
    const uint32_t lane16 = lane * 16;
    uint32_t b_off[NT];                                 // shuffled B: wave-uniform; row-major B: the lane's row and piece
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        if constexpr (BROW)
            b_off[t] = (uint32_t)((nt0 + t) * 16 + ld_row) * (uint32_t)p.ldb + ld_piece * 16;      // rows past n read as zero
        else
            b_off[t] = (uint32_t)min(nt0 + t, n_tiles - 1) * (uint32_t)k_tiles * 1024u;
    }
    // MX scales in the tiled layout of the dense kernels (mx_tiled_index): a pair of K blocks is one 128-wide K
    // step ks; lane (r16, kq) scales 32-block kq of its row, whose byte for step ks sits at
    // ((ks / 4 * nblk + blk) * 2 + (ks / 2) % 2) * 512 + ((4x + y) * 4 + kq) * 8 + jp * 4 + par * 2 + ks % 2
    // with, for row 16 i + r16 of a 64-row block, x = (2 i + r16 / 8) % 4, y = r16 % 4, jp = i / 2, par = (r16 / 4) % 2
    const auto rs_sa = make_rsrc((const uint8_t*)p.sfa + (long long)batch * p.sfa_batch, 0x7fffffffu);
    const auto rs_sb = make_rsrc((const uint8_t*)p.sfb + (long long)batch * p.sfb_batch, 0x7fffffffu);
    // offsets of row groups / weight tiles 1, 2, 3 of a 64-row block from group 0's, for a lane (see lane_off below)
    constexpr uint32_t MX_DELTA[4] = {0u, 256u, 4u, 260u};
    uint32_t mx_a[MT], mx_b[NT];
    int mx_nblk_a = 1, mx_nblk_b = 1;
    if constexpr (MODE == MODE_MXT || MODE == MODE_F4T) {
        auto lane_off = [&](int i) { return ((4 * ((2 * i + (r16 >> 3)) & 3) + (r16 & 3)) * 4 + kq) * 8 + (i >> 1) * 4 + ((r16 >> 2) & 1) * 2; };
        mx_nblk_a = (p.m + 63) >> 6;
        mx_nblk_b = (p.n + 63) >> 6;
#pragma unroll
        for (int g = 0; g < MT; ++g) {
            const int mt = min(m_tile_ * MT + g, ((p.m + 15) >> 4) - 1);
            // four groups are one 64-row block: constant distances from group 0 (rows past m stay inside the block)
            // (the distance goes into the scalar offset of the load: one lane offset for the four groups)
            mx_a[g] = MT == 4 ? (uint32_t)m_tile_ * 1024u + lane_off(0) : (uint32_t)(mt >> 2) * 1024u + lane_off(mt & 3);
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int nt = min(nt0 + t, n_tiles - 1);
            mx_b[t] = NT == 4 ? (uint32_t)n_group * 1024u + lane_off(0) : (uint32_t)(nt >> 2) * 1024u + lane_off(nt & 3);
        }
    }

    // block scales (1x128 for A, 128x128 for B; the reference's layout): a pair of K blocks is one 128-wide scale
    // group, lane (r16, .) needs sfa[group][its row] and, per weight tile, sfb[tile's 128-row block][group]
    uint32_t blk_a_off = 0;
    const auto rs_blk_a = make_rsrc((const float*)p.sfa + (long long)batch * p.sfa_batch,
                                    MODE == MODE_BLOCK ? ((uint32_t)(p.k / 128 - 1) * (uint32_t)p.stride_sfa + (uint32_t)p.m) * 4u : 0u);
    const float* blk_b;      // NT divides 8 and the tile groups start at multiples of NT: one 128-row block per workgroup
    if constexpr (MODE == MODE_BLOCK) {
        // sfa[group][row] through a descriptor over the whole array: one lane offset (the row), the row groups 64 bytes
        // apart, the K group scalar; rows past m read a neighbour's scale or zero and feed rows that are not stored
        blk_a_off = (uint32_t)(m0 + r16) * 4u;
        static_assert(MODE != MODE_BLOCK || 8 % NT == 0, "the weight tiles of a workgroup share their block scale");
        blk_b = (const float*)p.sfb + (long long)batch * p.sfb_batch + (long long)(nt0 >> 3) * p.stride_sfb;
    }

    // K blocks are consumed in pairs, eight consecutive pairs a round, one per wave: at any moment the eight waves
    // read 16 KiB in a row of each weight tile.  (Contiguous shares put the waves K/8 bytes apart, which for a
    // power-of-two K lands all of them, in every workgroup, on the same few memory channels.)
    const int pairs = (k_tiles + 1) >> 1;
    constexpr int PSTEP = FLAT_WAVES;

    v4f acc[MT][NT];
#pragma unroll
    for (int g = 0; g < MT; ++g)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[g][t] = v4f{0.f, 0.f, 0.f, 0.f};

    struct Frag {
        v4i a[2];               // MT = 1: the activation fragment itself
        v4i b[NT][2];
        int sa[MT], sb[NT];     // MX: the step's E8M0 byte of this lane's row and 32-block
        float fsa[MT], fsb;     // block scales of the pair's scale group
    };
    // MT > 1: the rows of one pair in flight (one register set: a pair's rows go to LDS before the next is asked for)
    v4i raw[MT][2];
    v4i raw_b[NT][2];          // BROW: the same for the rows of the weight tiles
    auto load_rows = [&](int pp) {
        // pieces 4 .. 7 are the second K block of the pair: past the end of K (an odd number of blocks) they get an
        // offset beyond the descriptor's extent instead of a branch, which reads as zero and touches no memory
        const uint32_t off = a_off[0] | (2 * pp + 1 < k_tiles ? 0u : kill_second);
#pragma unroll
        for (int g = 0; g < MT; ++g) {
            // (group g is 16 g rows on: a scalar offset, so that one lane offset serves every group)
            raw[g][0] = ld16(rs_a, off, pp * 128 + 16 * g * p.lda);
            raw[g][1] = ld16(rs_a, off, pp * 128 + (16 * g + 8) * p.lda);
        }
    };
    auto load_weight_rows = [&](int pp) {
        const uint32_t off = b_off[0] | (2 * pp + 1 < k_tiles ? 0u : kill_second);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            // (tile t is 16 t rows on: a scalar offset, one lane offset for every tile)
            raw_b[t][0] = ld16_nt(rs_b, off, pp * 128 + 16 * t * p.ldb);
            raw_b[t][1] = ld16_nt(rs_b, off, pp * 128 + (16 * t + 8) * p.ldb);
        }
    };
    // rows -> this wave's own LDS.  A wave's LDS operations complete in order, so the fragment reads that follow
    // see these writes, and these writes cannot pass the fragment reads of the pair before.
    auto stage_rows = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int g = 0; g < A_GROUPS; ++g) {
            stage[g * FLAT_STAGE_SLOTS + st_write] = raw[g][0];
            stage[g * FLAT_STAGE_SLOTS + st_write + 8] = raw[g][1];
        }
        if constexpr (BROW) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                stage[(A_GROUPS + t) * FLAT_STAGE_SLOTS + st_write] = raw_b[t][0];
                stage[(A_GROUPS + t) * FLAT_STAGE_SLOTS + st_write + 8] = raw_b[t][1];
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    auto load = [&](int pp, Frag& f) {
        const int kt0 = 2 * pp, kt1 = 2 * pp + 1;
        const uint32_t kill1 = kt1 < k_tiles ? 0u : 0x80000000u;      // reads as zero, see load_rows
        if constexpr (MT == 1) {
            f.a[0] = ld16(rs_a, a_off[0], kt0 * 64);
            f.a[1] = ld16(rs_a, a_off[0] | kill1, kt1 * 64);
        }
        int unit_a = 0, unit_b = 0;
        if constexpr (MODE == MODE_MXT) {
            unit_a = ((pp >> 2) * mx_nblk_a * 2 + ((pp >> 1) & 1)) * 512 + (pp & 1);
            unit_b = ((pp >> 2) * mx_nblk_b * 2 + ((pp >> 1) & 1)) * 512 + (pp & 1);
#pragma unroll
            for (int g = 0; g < MT; ++g) f.sa[g] = __builtin_amdgcn_raw_buffer_load_b8(rs_sa, mx_a[MT == 4 ? 0 : g], unit_a + (MT == 4 ? (int)MX_DELTA[g & 3] : 0), 0);
        }
        if constexpr (MODE == MODE_F4T) {
            // FP4: a pair of 64-byte blocks is two 128-element K steps, whose two scale bytes sit side by side
            unit_a = ((pp >> 1) * mx_nblk_a * 2 + (pp & 1)) * 512;
            unit_b = ((pp >> 1) * mx_nblk_b * 2 + (pp & 1)) * 512;
#pragma unroll
            for (int g = 0; g < MT; ++g) f.sa[g] = __builtin_amdgcn_raw_buffer_load_b16(rs_sa, mx_a[MT == 4 ? 0 : g], unit_a + (MT == 4 ? (int)MX_DELTA[g & 3] : 0), 0);
        }
        if constexpr (MODE == MODE_BLOCK) {
#pragma unroll
            for (int g = 0; g < MT; ++g)
                f.fsa[g] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs_blk_a, blk_a_off + 64u * g, pp * p.stride_sfa * 4, 0));
            f.fsb = blk_b[pp];
        }
        // (the scale bytes before the weights: loads complete in issue order, and pack_scales waits for these only)
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if constexpr (MODE == MODE_MXT) f.sb[t] = __builtin_amdgcn_raw_buffer_load_b8(rs_sb, mx_b[NT == 4 ? 0 : t], unit_b + (NT == 4 ? (int)MX_DELTA[t & 3] : 0), 0);
            if constexpr (MODE == MODE_F4T) f.sb[t] = __builtin_amdgcn_raw_buffer_load_b16(rs_sb, mx_b[NT == 4 ? 0 : t], unit_b + (NT == 4 ? (int)MX_DELTA[t & 3] : 0), 0);
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if constexpr (!BROW) {
                f.b[t][0] = ld16_nt(rs_b, lane16, b_off[t] + kt0 * 1024);
                f.b[t][1] = ld16_nt(rs_b, lane16 | kill1, b_off[t] + kt1 * 1024);
            }
        }
    };
    // MXFP8: the pair's scale bytes, four to a register (byte g % 4 / byte t, picked by the MFMA's op_sel): the
    // registers they arrived in are free for the next pair's before its loads are issued
    struct Packed { int a[(MT + 3) / 4], b; };
    auto pack_scales = [&](const Frag& f) {
        Packed q{};
        if constexpr (MODE == MODE_MXT) {
#pragma unroll
            for (int g = 0; g < MT; ++g) q.a[g >> 2] = (g & 3) ? q.a[g >> 2] | (f.sa[g] << (8 * (g & 3))) : f.sa[g];
            q.b = f.sb[0];
#pragma unroll
            for (int t = 1; t < NT; ++t) q.b |= f.sb[t] << (8 * t);
#pragma unroll
            for (int w = 0; w < (MT + 3) / 4; ++w) asm volatile("" : "+v"(q.a[w]));
            asm volatile("" : "+v"(q.b));
        }
        return q;
    };
    auto mma = [&](const Frag& f, const Packed q) {
        v4i blo[NT], bhi[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if constexpr (BROW) {
                blo[t] = stage[(A_GROUPS + t) * FLAT_STAGE_SLOTS + st_read];
                bhi[t] = stage[(A_GROUPS + t) * FLAT_STAGE_SLOTS + st_read + 4 * 18];
            } else {
                blo[t] = f.b[t][0];
                bhi[t] = f.b[t][1];
            }
        }
#pragma unroll
        for (int g = 0; g < MT; ++g) {
            v4i alo, ahi;
            if constexpr (MT == 1) {
                alo = f.a[0];
                ahi = f.a[1];
            } else {
                alo = stage[g * FLAT_STAGE_SLOTS + st_read];
                ahi = stage[g * FLAT_STAGE_SLOTS + st_read + 4 * 18];
            }
            const v8i fa = v8i{alo.x, alo.y, alo.z, alo.w, ahi.x, ahi.y, ahi.z, ahi.w};
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const v8i fb = v8i{blo[t].x, blo[t].y, blo[t].z, blo[t].w, bhi[t].x, bhi[t].y, bhi[t].z, bhi[t].w};
                if constexpr (MODE == MODE_BF16) {
                    // bf16 weights: a 1 KiB block is 16 rows x 32 bf16, one 16x16x32 MFMA operand
                    acc[g][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, blo[t]),
                                                                        __builtin_bit_cast(v8bf, alo), acc[g][t], 0, 0, 0);
                    acc[g][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, bhi[t]),
                                                                        __builtin_bit_cast(v8bf, ahi), acc[g][t], 0, 0, 0);
                } else if constexpr (MODE == MODE_BLOCK) {
                    // each 128-wide K group yields a partial tile that is rescaled into the running sum
                    const v4f part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb, fa, v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                    acc[g][t] += part * (f.fsa[g] * f.fsb);
                } else if constexpr (MODE == MODE_F4T) {
                    // packed E2M1: a 64-byte block is 128 elements, one FP4 MFMA; op_sel picks the block's scale byte
                    acc[g][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                        (v8i{blo[t].x, blo[t].y, blo[t].z, blo[t].w, 0, 0, 0, 0}), (v8i{alo.x, alo.y, alo.z, alo.w, 0, 0, 0, 0}),
                        acc[g][t], 4, 4, 0, f.sb[t], 0, f.sa[g]);
                    acc[g][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                        (v8i{bhi[t].x, bhi[t].y, bhi[t].z, bhi[t].w, 0, 0, 0, 0}), (v8i{ahi.x, ahi.y, ahi.z, ahi.w, 0, 0, 0, 0}),
                        acc[g][t], 4, 4, 1, f.sb[t], 1, f.sa[g]);
                } else if constexpr (MODE == MODE_MXT) {
                    acc[g][t] = mfma_mx_bytes(fb, fa, acc[g][t], t, q.b, g & 3, q.a[g >> 2]);
                } else {
                    acc[g][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb, fa, acc[g][t], 0, 0, 0, 0, 0, 0);
                }
            }
        }
    };

    {
        Frag f0, f1;
        constexpr bool STAGING = MT > 1 || BROW;
        auto load_staged = [&](int q) {
            if constexpr (MT > 1) load_rows(q);
            if constexpr (BROW) load_weight_rows(q);
        };
        // Round j of the K walk covers pairs 8 j .. 8 j + 7, one per wave; the wave takes slot (wave + 3 j) % 8 of its
        // round.  A fixed slot would advance every wave by exactly 16 KiB per round, and memory channels repeat with
        // a period that divides 16 KiB: each wave would then sit on the same few channels for its whole life, all
        // waves of all workgroups aliasing onto one another (16 x 16384 x 7168: 20.0 us with fixed slots, 18.9 us
        // rotating).  The wave starts at a round that depends on the workgroup and wraps around, so that workgroups
        // running side by side are at different K offsets as well: with rows (or weight tiles) a power of two apart
        // they would otherwise all sit on the same memory channels at any moment.
        const int rounds = (pairs + PSTEP - 1) / PSTEP;
        auto pair_of = [&](int j) { return ((wave + 3 * j) & (PSTEP - 1)) + PSTEP * j; };
        // the last round may be partial: this wave has a pair in it only if its slot there exists
        const int count = pair_of(rounds - 1) < pairs ? rounds : rounds - 1;
        // (the same start for the workgroups of one group of weight tiles: those read the weights together, through L2)
        // (a multiplicative hash of the group index scaled into [0, count): no division in front of the first load)
        int at = (int)((((uint32_t)n_group * 40503u) & 0xffffu) * (uint32_t)count >> 16);
        auto next_of = [&](int j) { return j + 1 == count ? 0 : j + 1; };
        int left = count;
        if (count > 0) {
            load_staged(pair_of(at));
            load(pair_of(at), f0);
        }
        if constexpr (ROUNDS == 1) fetch_scales(0);
        // two register stages, loads of the next pair in flight while the current one is used
        while (left > 0) {
            if constexpr (STAGING) stage_rows();
            at = next_of(at);
            const Packed q0 = pack_scales(f0);
            if (left > 1) {
                load_staged(pair_of(at));
                load(pair_of(at), f1);
            }
            mma(f0, q0);
            if (--left == 0) break;
            if constexpr (STAGING) stage_rows();
            at = next_of(at);
            const Packed q1 = pack_scales(f1);
            if (left > 1) {
                load_staged(pair_of(at));
                load(pair_of(at), f0);
            }
            mma(f1, q1);
            if (--left == 0) break;
        }
    }

    // the partial tiles of the eight K shares are summed through LDS (the same memory as the staging above)
    v4f* red = (v4f*)smem;
#pragma unroll
    for (int r = ROUNDS == 1 ? 1 : 0; r < ROUNDS; ++r) fetch_scales(r);      // in flight during the reduction
    constexpr int PER_ROUND = TILES < FLAT_WAVES ? TILES : FLAT_WAVES;
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
        if (MT > 1 || BROW || r > 0) __syncthreads();
#pragma unroll
        for (int j = 0; j < PER_ROUND; ++j) {
            const int c = r * FLAT_WAVES + j;
            if (c < TILES) red[(wave * PER_ROUND + j) * 64 + lane] = acc[c / NT][c % NT];
        }
        __syncthreads();
        if (finisher[r]) {
            v4f s = red[(0 * PER_ROUND + wave) * 64 + lane];
#pragma unroll
            for (int w = 1; w < FLAT_WAVES; ++w) s += red[(w * PER_ROUND + wave) * 64 + lane];
            s *= sb[r] * sa[r];
            const long long ci = c_batch_off + (long long)cm[r] * ldc + cn[r];
            if constexpr (CDT == C_BF16) {
                unsigned short* dst = (unsigned short*)p.c + ci;
                if ((ldc & 3) == 0 && (((uintptr_t)p.c + 2 * c_batch_off) & 7) == 0) {
                    *(v2i*)dst = v2i{bf16x2_bits(s.x, s.y), bf16x2_bits(s.z, s.w)};
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
}

}  // namespace a8w8
