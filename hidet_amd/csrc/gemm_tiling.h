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

// XOR keys of the LDS chunk swizzle for operand tiles with 128-byte rows (8 chunks of 16 bytes): chunk c of tile row r
// is stored at position c ^ key(r) of that row.
//
// The LDS has 64 banks of 4 bytes; a 16-byte-per-lane read (ds_read_b128) is served 16 lanes per cycle, in the groups
// {0-3, 12-15, 20-23, 24-27}, {4-7, 8-11, 16-19, 28-31} and the same two shifted by 32 (measured with
// SQ_LDS_BANK_CONFLICT on access patterns built for the purpose). A group is conflict-free when its 16 lanes hit 16
// different 16-byte bank groups, (row % 2) * 8 + position.
//
// MFMA operand fragments are read by lane (g, r) = (lane / 16, lane % 16) at row r and chunk g * step + const:
//   step 1 (f16/bf16 16x16x32: 8 halves per lane)      -> key r % 8 is conflict-free,
//   step 2 (fp8 16x16x128: 32 bytes = 2 chunks per lane) -> key (r % 8) ^ (r / 8 % 2) is.
// Each key fails (2-way conflict on every read) on the other pattern.
__host__ __device__ constexpr int lds_swizzle_key_step1(int row) { return row & 7; }
__host__ __device__ constexpr int lds_swizzle_key_step2(int row) { return (row & 7) ^ ((row >> 3) & 1); }

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

struct GemmRegion {
    int row_begin, col_begin, rows, cols;
};

__device__ __forceinline__ GemmRegion gemm_region_of_xcd(int tiles_m, int tiles_n, int xm, int xn, int xcd) {
    const int xr = xcd / xn, xc = xcd % xn;
    const int r_begin = (tiles_m * xr) / xm, r_end = (tiles_m * (xr + 1)) / xm;
    const int c_begin = (tiles_n * xc) / xn, c_end = (tiles_n * (xc + 1)) / xn;
    return GemmRegion{r_begin, c_begin, r_end - r_begin, c_end - c_begin};
}

// Tile (row, column) number `local` of a region in panel order; false past the end of the region.
__device__ __forceinline__ bool gemm_tile_of_region(const GemmRegion &reg, int local, int *tile_m, int *tile_n) {
    const int rr = reg.rows, rc = reg.cols;
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
    *tile_m = reg.row_begin + row;
    *tile_n = reg.col_begin + col;
    return true;
}

// Tile (row, column) of this workgroup; false when it has none (its XCD's region is smaller than the largest).
__device__ __forceinline__ bool gemm_tile_of_block(int tiles_m, int tiles_n, int xm, int xn, int *tile_m, int *tile_n) {
    const GemmRegion reg = gemm_region_of_xcd(tiles_m, tiles_n, xm, xn, blockIdx.x & 7);
    return gemm_tile_of_region(reg, blockIdx.x >> 3, tile_m, tile_n);
}

// Tiles XCD `xcd` owns (host-side twin of gemm_region_of_xcd).
inline int gemm_region_tiles(const GemmTiling &t, int xcd) {
    const int xr = xcd / t.xn, xc = xcd % t.xn;
    const int rows = (t.tiles_m * (xr + 1)) / t.xm - (t.tiles_m * xr) / t.xm;
    const int cols = (t.tiles_n * (xc + 1)) / t.xn - (t.tiles_n * xc) / t.xn;
    return rows * cols;
}

// Tail split: the tiles of an XCD that do not fill a whole round of `concurrent` workgroups are cut into K ranges.
struct GemmTail {
    int parts;      // K ranges per tail tile (1 = no split)
    int max_tiles;  // most tail tiles any XCD has: stride of the per-XCD blocks of fix-up slots
    int64_t grid;   // workgroups to launch
};

// K ranges are worth their fix-up traffic only while an XCD has fewer tiles than CUs (32): then as many parts (up to
// max_parts) as keep the busiest XCD at one workgroup per CU. With whole rounds of workgroups in flight the kernels
// run at the chip's power limit and a shorter last round buys nothing (measured), so the tail stays whole.
inline GemmTail make_gemm_tail(const GemmTiling &t, int concurrent, int max_parts) {
    GemmTail tail{1, 0, t.grid()};
    constexpr int kCusPerXcd = 32;
    if (t.region_tiles >= concurrent || t.region_tiles == 0) return tail;
    for (int x = 0; x < 8; ++x) {
        const int n = gemm_region_tiles(t, x);
        if (n > tail.max_tiles) tail.max_tiles = n;
    }
    int parts = kCusPerXcd / t.region_tiles;
    if (parts > max_parts) parts = max_parts;
    tail.parts = parts < 1 ? 1 : parts;
    return tail;
}

// Workgroups per XCD x 8 once the tails are cut into tail.parts ranges.
inline int64_t gemm_grid_with_tail(const GemmTiling &t, int concurrent, const GemmTail &tail) {
    if (tail.parts <= 1) return t.grid();
    int64_t most = 0;
    for (int x = 0; x < 8; ++x) {
        const int n = gemm_region_tiles(t, x);
        const int whole = (n / concurrent) * concurrent;
        const int64_t items = whole + int64_t(n - whole) * tail.parts;
        if (items > most) most = items;
    }
    return 8 * most;
}

}  // namespace qmm
