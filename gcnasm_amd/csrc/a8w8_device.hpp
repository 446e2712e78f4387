// Device-side building blocks shared by the gfx950 A8W8 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace a8w8 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned short v4u16 __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

#define A8W8_DEV __device__ __forceinline__
#define A8W8_LDS __attribute__((address_space(3)))

// MODE_BF16: A and B hold bf16 (the a16w16 sibling), no scales; the kernels see them as byte matrices of 2k columns
// MODE_F4 / MODE_F4T: A and B hold packed E2M1 (MXFP4: two elements per byte, even K in the low nibble) with
// row-major / tiled E8M0 scales; the kernels see byte matrices of k/2 columns
enum : int { MODE_TENSOR = 0, MODE_ROWCOL = 1, MODE_BLOCK = 2, MODE_MX = 3, MODE_MXT = 4, MODE_BF16 = 5, MODE_F4 = 6, MODE_F4T = 7 };

// Byte position of the E8M0 exponent of (row, 32-wide K block kblk) in the tiled MX scale layout
//   [K/512][ceil(rows/64)][pair of K steps: 2][r16: 16][g: 4][jp: 2][par: 2][s: 2]       (1 byte each)
// where, inside a 64-row block, row = 32 jp + 8 (r16 >> 2) + 4 par + (r16 & 3) is the row that lane
// r16 supplies to MFMA tile 2 jp + par of the block, g = kblk & 3 is the 32-block inside a 128-wide
// K step and s the step inside the pair.  The eight bytes of (r16, g) are what one lane of the
// scaled MFMA needs for two K steps of a 64-row block: two dwords, each holding two tiles x two
// steps, selected per instruction through op_sel.  A 64-row block takes 1 KiB per 512 of K.
__host__ __device__ inline size_t mx_tiled_index(int rows, int row, int kblk)
{
    const int nblk = (rows + 63) >> 6, blk = row >> 6, rr = row & 63;
    const int jp = rr >> 5, x = (rr >> 3) & 3, par = (rr >> 2) & 1, y = rr & 3;
    const int g = kblk & 3, s = (kblk >> 2) & 1, pair = (kblk >> 3) & 1;
    return ((((size_t)(kblk >> 4) * nblk + blk) * 2 + pair) * 64 + (4 * x + y) * 4 + g) * 8 + jp * 4 + par * 2 + s;
}
__host__ __device__ inline size_t mx_tiled_bytes(int rows, int k)
{
    return (size_t)((k + 511) >> 9) * ((rows + 63) >> 6) * 1024;
}

enum : int { C_BF16 = 0, C_FP32 = 1 };

// Kernel parameters of the dense and flat GEMMs (strides in elements, as in the ABI).
struct GemmParams {
    const uint8_t* a;
    const uint8_t* b;
    void* c;
    const void* sfa;
    const void* sfb;
    int m, n, k;
    int lda, ldb, ldc;
    long long a_batch, b_batch, c_batch, sfa_batch, sfb_batch;
    int stride_sfa, stride_sfb;
    int tiles_m, tiles_n;
    // log2 of the byte distance between consecutive 128-wide K steps of a row of B: 7 for row-major B, 11 for B in
    // the a8w8_preshuffle_b layout (two 1 KiB blocks per step; ldb = k there, so that 16 r rows are 16 r * ldb bytes)
    int b_kshift;
};

// Raw buffer descriptor over [base, base + bytes): dword 3 = 0x00020000 selects the raw
// 32-bit data format used for untyped loads on gfx9-family hardware.
A8W8_DEV __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

// Byte offset, inside B, of the 16-byte K piece at `piece_bytes` (0, 16, .. 112) of the first K step of row `row`.
// Pre-shuffled B [n/16][k/64][4][16][16 B]: the piece's 64-wide K block, its quarter of the block, the row's slot.
A8W8_DEV int b_lane_offset(const GemmParams& p, int row, int piece_bytes)
{
    if (p.b_kshift == 7) return row * p.ldb + piece_bytes;
    return (row >> 4) * (p.k << 4) + ((piece_bytes >> 6) << 10) + (((piece_bytes >> 4) & 3) << 8) + ((row & 15) << 4);
}
// Extent of one batch entry of B for its buffer descriptor (rows past n read as zero in both layouts).
A8W8_DEV uint32_t b_extent_bytes(const GemmParams& p)
{
    return p.b_kshift == 7 ? (uint32_t)(p.n - 1) * p.ldb + p.k : (uint32_t)p.n * p.k;
}

// 16 bytes per lane straight from global memory into LDS.  The hardware places lane i's
// data at lds_base + 16*i, so lds_base must be wave-uniform.
A8W8_DEV void load_to_lds_16(__amdgpu_buffer_rsrc_t rsrc, A8W8_LDS void* lds_base, int voffset, int soffset)
{
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, lds_base, 16, voffset, soffset, 0, 0);
}

// C stores stay ordinary write-back stores: each lane writes 8 or 16 bytes and L2 merges the
// pieces of a line; non-temporal stores of such pieces were measured 30% slower end to end.
#ifndef A8W8_C_STORE_NT
#define A8W8_C_STORE_NT 0
#endif
#if A8W8_C_STORE_NT
#define A8W8_STORE_C(ptr, val) __builtin_nontemporal_store((val), (ptr))
#else
#define A8W8_STORE_C(ptr, val) (*(ptr) = (val))
#endif

// 16 bytes of a whole C tile through a buffer descriptor over the tile.
// WRITE_THROUGH: the store carries the sc1 bit: the line is written through to memory as it is stored instead of
// waiting in this XCD's L2 for the write-back at the end of the kernel, which otherwise delays the next launch (2 us
// less per launch measured for a 32 MiB bf16 C).  Only for stores whose lanes together cover whole 64-byte pieces
// of a line, as store_c_lines arranges them; interleaved 16-byte
// pieces have to be merged by L2 first (written through, a 8192 x 8192 fp32 C took 557 us instead of 452).
// A 16-byte buffer store reads its data registers for a few cycles after it issues.  The compiler keeps the next
// write to them at a distance only when the scalar-offset field holds no register; with a register there, fp32
// outputs stored straight from the accumulators came out overwritten, in some lanes, by the scale products the next
// instruction put into the same registers.  Hence the two idle cycles, in a statement that keeps `data` alive across
// them (the build checks that they directly follow every such store).
template <bool WRITE_THROUGH>
A8W8_DEV void store_c_16(__amdgpu_buffer_rsrc_t rsrc, v4i data, int lane_offset, int scalar_offset)
{
#if defined(A8W8_ABLATE_STORE_INSTRUCTIONS)
    asm volatile("" ::"v"(lane_offset), "s"(scalar_offset), "s"(rsrc));      // measurement: everything but the store itself
#elif defined(A8W8_STORE_AUX)
    __builtin_amdgcn_raw_buffer_store_b128(data, rsrc, lane_offset, scalar_offset, A8W8_STORE_AUX);      // measurement: cache policy bits
#else
    __builtin_amdgcn_raw_buffer_store_b128(data, rsrc, lane_offset, scalar_offset, WRITE_THROUGH ? 16 : 0);
#endif
    asm volatile("s_nop 1" ::"v"(data));
}

// The value of the lane eight places away inside the lane's row of 16 (DPP row_ror:8).
A8W8_DEV int from_lane_8_apart(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, 0x128, 0xf, 0xf, false);
}

// The two 16-byte halves `lo`, `hi` of the eight consecutive fp32 columns a lane holds of one row of a whole C tile
// (`hi` DISTANCE = 16 bytes after `lo`), or two bf16 pieces of the row side by side (DISTANCE 64).  Stored as they are,
// each store of a wave would cover every other 16 bytes (bf16: 64-byte halves) of 16 rows.  Instead
//  1. the lanes of rows r and r + 8 (of the 16 a wave's store covers) exchange halves (DPP row_ror:8), so that one store
//     holds rows 0 .. 7 and the other rows 8 .. 15, each row as one contiguous 128-byte line: whole lines, which can take
//     the write-through path;
//  2. (BY_LANE) the 16-byte units of each store are moved between the lanes (ds_bpermute, four per store) so that
//     CONSECUTIVE LANES hold consecutive 16 bytes of a line: lane L writes piece L % 8 of row L / 8.  The memory pipeline
//     takes a store's lanes in order, and a store whose neighbouring lanes lie in different rows occupies it 2.7 times as
//     long as one whose lanes run along the lines (26.8 against 10.5 ns per 1 KiB store and compute unit, measured with
//     nothing else running).  The eight-wave kernel gains 1.5-2% from it; the four-wave kernel, whose workgroups all
//     reach their stores within the same few microseconds and are then bound by what the whole chip can store at once
//     (about 30 ns per store and compute unit either way), does not, and leaves step 2 out.
// upper: the lane's row index within the 16 is 8 or more; source_low / _high: c_line_source of the lane for the two stores;
// lane_offset_low / _high: the lane's place in the first / second store (c_line_offsets, per tile).
template <bool BY_LANE>
A8W8_DEV void store_c_lines(__amdgpu_buffer_rsrc_t rsrc, v4i lo, v4i hi, bool upper, int source_low, int source_high,
                            int lane_offset_low, int lane_offset_high, int scalar_offset)
{
    const v4i r = {from_lane_8_apart(hi.x), from_lane_8_apart(hi.y), from_lane_8_apart(hi.z), from_lane_8_apart(hi.w)};
    v4i first = upper ? r : lo, second = upper ? lo : r;
    if constexpr (BY_LANE) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            first[e] = __builtin_amdgcn_ds_bpermute(source_low, first[e]);
            second[e] = __builtin_amdgcn_ds_bpermute(source_high, second[e]);
        }
    }
    store_c_16<true>(rsrc, first, lane_offset_low, scalar_offset);
    store_c_16<true>(rsrc, second, lane_offset_high, scalar_offset);
}
// After step 1 lane 16 g + r16 holds, of row r16 % 8 of each store, a 16-byte piece of the row's line: in the first
// store piece 4 u + g (bf16 pairs, DISTANCE 64: the line is two 64-byte halves of four pieces) or 2 g + u (fp32, DISTANCE
// 16) with u = r16 / 8, in the second store the same with 1 - u.  The byte address (lane x 4) of the lane that holds what
// lane `lane` is to write, piece lane % 8 of row lane / 8, in the first (second = false) or second store.
template <int DISTANCE, bool BY_LANE>
A8W8_DEV int c_line_source(int lane, bool second)
{
    if constexpr (!BY_LANE) return 4 * lane;
    const int row = lane >> 3, piece = lane & 7;
    const int g = DISTANCE == 64 ? (piece & 3) : (piece >> 1), u = DISTANCE == 64 ? (piece >> 2) : (piece & 1);
    return 4 * (16 * g + 8 * (second ? 1 - u : u) + row);
}
// the row (0 .. 7) of the 16 that `lane` writes in the first store (the second: 8 more)
template <bool BY_LANE>
A8W8_DEV int c_line_row(int lane)
{
    return BY_LANE ? lane >> 3 : lane & 7;
}
// The two lane offsets of store_c_lines: row_low / row_high = byte offsets of rows c_line_row(lane) and c_line_row(lane) + 8
// of the 16, col = byte offset of the line inside a row.  By lane: piece lane % 8 of the line.  Otherwise (r16, g = lane % 16,
// lane / 16): the lane's own piece g, the halves DISTANCE apart.
template <int DISTANCE, bool BY_LANE>
A8W8_DEV void c_line_offsets(int lane, int row_low, int row_high, int col, int& lane_offset_low, int& lane_offset_high)
{
    if constexpr (BY_LANE) {
        lane_offset_low = (int)((uint32_t)row_low + (uint32_t)(col + 16 * (lane & 7)));
        lane_offset_high = (int)((uint32_t)row_high + (uint32_t)(col + 16 * (lane & 7)));
    } else {
        const bool upper = (lane & 15) >= 8;
        const int piece = (lane >> 4) * (DISTANCE == 64 ? 16 : 32);
        lane_offset_low = (int)((uint32_t)row_low + (uint32_t)(col + piece + (upper ? DISTANCE : 0)));
        lane_offset_high = (int)((uint32_t)row_high + (uint32_t)(col + piece + (upper ? 0 : DISTANCE)));
    }
}

// Barrier without the wait for every outstanding load that __syncthreads() implies: the pipelined kernels
// keep direct-to-LDS loads in flight across it and place their own s_waitcnt.
#define A8W8_RAW_BARRIER() asm volatile("s_barrier" ::: "memory")

A8W8_DEV int wave_uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// fp32 -> bf16 bits, round to nearest even, through the hardware convert.
A8W8_DEV unsigned short bf16_bits(float f)
{
    __bf16 h = (__bf16)f;
    return __builtin_bit_cast(unsigned short, h);
}
// Two at once, `lo` in the low half of the word: one v_cvt_pk_bf16_f32.  (Built from two bf16_bits the compiler
// converts each value with an instruction of its own and joins them with a shift and an or: six instructions for
// two values, which in an epilogue that runs beside the MFMAs is what the MFMAs end up waiting for.)
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
A8W8_DEV int bf16x2_bits(float lo, float hi)
{
    return __builtin_bit_cast(int, __builtin_convertvector((v2f{lo, hi}), v2bf));
}

}  // namespace a8w8
