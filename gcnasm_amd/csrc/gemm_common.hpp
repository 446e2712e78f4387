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

// The same mapping for the persistent kernels, which look tiles up at every tile change, where nothing hides the
// lookup: every division is by a value the host knows, so the host passes floor(2^32 / d) for each of them and the
// kernel divides with one multiply and one correction (exact for 0 <= n < 2^31 and any d >= 1: the estimate
// mulhi(n, floor(2^32 / d)) is the quotient or one less).  Measured against run-time divisors: 0.25% of the MXFP8 8192^3
// launch (four tiles per workgroup), 1-2% of block-scale 4096 x 7168 x 2048 (two tiles of 16 K steps).
struct TileMap {
    int tiles_m, tiles_n;
    int tiles;                 // tiles_m * tiles_n
    int per_group;             // 8 * tiles_n: the tiles of eight tile rows
    int rem;                   // tiles_m % 8: tile rows of the last group when it is not a full one (0: none)
    uint32_t inv_tiles, inv_per_group, inv_rem;      // floor(2^32 / d) of the three divisors (d = 1: 2^32 - 1)
};
__host__ __device__ inline uint32_t tile_map_inverse(int d)
{
    return d <= 1 ? 0xFFFFFFFFu : (uint32_t)((1ull << 32) / (uint32_t)d);
}
__host__ inline TileMap make_tile_map(int tiles_m, int tiles_n)
{
    TileMap t;
    t.tiles_m = tiles_m; t.tiles_n = tiles_n;
    t.tiles = tiles_m * tiles_n;
    t.per_group = 8 * tiles_n;
    t.rem = tiles_m % 8;
    t.inv_tiles = tile_map_inverse(t.tiles);
    t.inv_per_group = tile_map_inverse(t.per_group);
    t.inv_rem = tile_map_inverse(t.rem);
    return t;
}
A8W8_DEV int div_by_known(int n, int d, uint32_t inv)
{
    int q = (int)__umulhi((uint32_t)n, inv);
    if (n - q * d >= d) ++q;
    return q;
}
// work item (batch entry, tile) -> batch entry and tile coordinates
A8W8_DEV void tile_of_item(const TileMap& t, int item, int& batch, int& tm, int& tn)
{
    batch = div_by_known(item, t.tiles, t.inv_tiles);
    const int bid = item - batch * t.tiles;
    int id = bid;
    if ((t.tiles & 7) == 0) id = (bid & 7) * (t.tiles >> 3) + (bid >> 3);
    const int group = div_by_known(id, t.per_group, t.inv_per_group);
    const int first_m = group * 8;
    const int in_group = id - group * t.per_group;
    if (t.tiles_m - first_m >= 8) {
        tn = in_group >> 3;
        tm = first_m + (in_group & 7);
    } else {
        tn = div_by_known(in_group, t.rem, t.inv_rem);
        tm = first_m + in_group - tn * t.rem;
    }
}

}  // namespace a8w8
