// Workgroup -> output tile mapping for the tiled GEMM kernels.
//
// Workgroups are dealt round-robin to the 8 XCDs (blockIdx % 8), each with its own L2. The tile grid is cut into
// xm x xn rectangular regions (xm * xn == 8), one per XCD, and inside a region the tiles are ordered in panels of
// kPanelCols tile columns, row-major within a panel. The workgroups an XCD runs at the same time are consecutive in
// that order, so they cover a compact block of the region (8 x 4 tiles for 32 CUs): per k-step they pull
// rows + cols operand slices into the L2 instead of the (all rows + 2 columns) a column-major order would.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace qmm {

struct GemmTiling {
    int tiles_m, tiles_n;
    int xm, xn;         // XCD grid
    int region_tiles;   // largest number of tiles any XCD owns
    int64_t grid() const { return int64_t(8) * region_tiles; }
};

constexpr int kPanelCols = 4;

// `concurrent` = workgroups one XCD runs at a time (32 CUs x workgroups per CU).
inline GemmTiling make_gemm_tiling(int tiles_m, int tiles_n, int concurrent) {
    GemmTiling best{tiles_m, tiles_n, 1, 8, 0};
    int64_t best_cost = -1;
    for (int xm = 1; xm <= 8; xm *= 2) {
        const int xn = 8 / xm;
        const int rr = (tiles_m + xm - 1) / xm, rc = (tiles_n + xn - 1) / xn;
        // rounds of workgroups on the busiest XCD first, then the operand slices one round pulls into its L2,
        // then the tile count of the busiest XCD
        const int rounds = (rr * rc + concurrent - 1) / concurrent;
        const int batch_rows = rr < concurrent / kPanelCols ? rr : concurrent / kPanelCols;
        int batch_cols = (concurrent + batch_rows - 1) / batch_rows;
        if (batch_cols > rc) batch_cols = rc;
        const int64_t cost = (int64_t(rounds) * 4096 + batch_rows + batch_cols) * 65536 + int64_t(rr) * rc;
        if (best_cost < 0 || cost < best_cost) {
            best_cost = cost;
            best.xm = xm;
            best.xn = xn;
            best.region_tiles = rr * rc;
        }
    }
    return best;
}

// Tile (row, column) of this workgroup; false when it has none (its XCD's region is smaller than the largest).
__device__ __forceinline__ bool gemm_tile_of_block(int tiles_m, int tiles_n, int xm, int xn, int *tile_m, int *tile_n) {
    const int xcd = blockIdx.x & 7;
    const int local = blockIdx.x >> 3;
    const int xr = xcd / xn, xc = xcd % xn;
    const int r_begin = (tiles_m * xr) / xm, r_end = (tiles_m * (xr + 1)) / xm;
    const int c_begin = (tiles_n * xc) / xn, c_end = (tiles_n * (xc + 1)) / xn;
    const int rr = r_end - r_begin, rc = c_end - c_begin;
    if (local >= rr * rc) return false;
    const int full_panels = rc / kPanelCols;
    const int full_tiles = full_panels * rr * kPanelCols;
    int row, col;
    if (local < full_tiles) {
        const int panel = local / (rr * kPanelCols), rem = local % (rr * kPanelCols);
        row = rem / kPanelCols;
        col = panel * kPanelCols + rem % kPanelCols;
    } else {
        const int rem = local - full_tiles, w = rc - full_panels * kPanelCols;
        row = rem / w;
        col = full_panels * kPanelCols + rem % w;
    }
    *tile_m = r_begin + row;
    *tile_n = c_begin + col;
    return true;
}

}  // namespace qmm
