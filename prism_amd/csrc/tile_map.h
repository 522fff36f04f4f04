// Workgroup id -> output tile, shared by the MFMA GEMM kernels.
//
// The role of the reference's persistent-kernel Schedule (super-tiles of
// 16 x 8 output tiles for L2 locality, evals/h100_bench/utils.cuh:277-307),
// recast for a chip whose 256 CUs sit in 8 XCDs with one L2 each and share a
// memory-side cache in front of HBM. The dispatcher hands out workgroup ids in
// order and deals consecutive ids to the XCDs round-robin, so:
//   * 256 consecutive ids (one tile per CU) form a super-block of 16 x 16
//     tiles; super-blocks advance along n, so the workgroups resident on the
//     chip at any time need 16 A panels and about 16 B panels from HBM instead
//     of a separate set per XCD;
//   * inside a super-block the ids of one XCD (every 8th id) cover an 8 x 4
//     patch, which re-uses 8 A panels and 4 B panels from that XCD's L2.
// Super-blocks at the edge of the grid are clipped; inside a clipped block the
// same construction runs on the smaller rectangle (every "XCD" owns a
// contiguous run of tile numbers, tile numbers walk the rectangle in
// column-major strips kGroupM tiles tall), so the map is a bijection for any
// grid.
#pragma once

namespace prism {

constexpr int kXcds = 8;
constexpr int kGroupM = 8;  // rows of tiles in one XCD's patch
constexpr int kSuper = 16;  // super-block edge, in tiles

__host__ __device__ __forceinline__ void xcd_tile_coords(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
    // Which super-block: rows of super-blocks hold kSuper * tiles_n tiles each (the last one fewer).
    const int sb_m = pid / (kSuper * tiles_n);
    const int in_row = pid - sb_m * kSuper * tiles_n;
    const int h = (tiles_m - sb_m * kSuper < kSuper) ? (tiles_m - sb_m * kSuper) : kSuper;
    const int last_n = (tiles_n - 1) / kSuper;
    int sb_n = in_row / (h * kSuper);
    if (sb_n > last_n) sb_n = last_n;
    const int w = (tiles_n - sb_n * kSuper < kSuper) ? (tiles_n - sb_n * kSuper) : kSuper;
    const int p = in_row - sb_n * h * kSuper;

    // Inside the h x w block.
    const int total = h * w;
    const int per = total / kXcds, rem = total % kXcds;
    const int xcd = p % kXcds, local = p / kXcds;
    const int logical = (xcd < rem) ? xcd * (per + 1) + local
                                    : rem * (per + 1) + (xcd - rem) * per + local;
    const int width = kGroupM * w;
    const int group = logical / width;
    const int first_m = group * kGroupM;
    const int group_rows = (h - first_m < kGroupM) ? (h - first_m) : kGroupM;
    const int in_group = logical % width;
    tm = sb_m * kSuper + first_m + in_group % group_rows;
    tn = sb_n * kSuper + in_group / group_rows;
}

}  // namespace prism
