// Workgroup id -> output tile, shared by the MFMA GEMM kernels.
//
// The role of the reference's persistent-kernel Schedule (super-tiles of
// 16 x 8 output tiles for L2 locality, evals/h100_bench/utils.cuh:277-307),
// recast for a chip whose 256 CUs sit in 8 XCDs with one L2 each: the
// dispatcher deals consecutive workgroup ids to the XCDs round-robin, so the id
// is first turned into (xcd, position within that xcd); every XCD then owns a
// contiguous run of "logical" tile ids, and logical ids walk the tile grid in
// column-major strips kGroupM tiles tall. The ~64 workgroups resident on one
// XCD thus cover a compact patch of C and re-use A and B panels from its L2.
#pragma once

namespace prism {

constexpr int kXcds = 8;
constexpr int kGroupM = 8;

__host__ __device__ __forceinline__ void xcd_tile_coords(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int total = tiles_m * tiles_n;
    const int per = total / kXcds, rem = total % kXcds;
    const int xcd = pid % kXcds, local = pid / kXcds;
    const int logical = (xcd < rem) ? xcd * (per + 1) + local
                                    : rem * (per + 1) + (xcd - rem) * per + local;
    const int width = kGroupM * tiles_n;
    const int group = logical / width;
    const int first_m = group * kGroupM;
    const int group_rows = (tiles_m - first_m < kGroupM) ? (tiles_m - first_m) : kGroupM;
    const int in_group = logical % width;
    tm = first_m + in_group % group_rows;
    tn = in_group / group_rows;
}

}  // namespace prism
