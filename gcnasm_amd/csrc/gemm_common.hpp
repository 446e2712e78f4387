// What the dense A8W8 GEMM kernels for gfx950 share: the 256 x 256 x 128 workgroup tile of the
// pipelined kernels (gemm_persist.hpp: 8 waves, 64 x 128 per wave; gemm_wide.hpp: 4 waves,
// 128 x 128 per wave), its LDS budget, and the workgroup-id -> tile mapping.
//
// Data path of every kernel: A and B tiles go global -> LDS with 16-byte direct-to-LDS buffer
// loads into 128-byte LDS rows (one K step of one matrix row) whose 16-byte slots are
// XOR-swizzled on the global-address side (the direct-to-LDS write itself is always
// wave-linear) and un-swizzled by the readers, which keeps the 64-lane ds_read_b128 free of
// bank conflicts.
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

}  // namespace a8w8
