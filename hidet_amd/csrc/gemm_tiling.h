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

#include "common.h"

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

__host__ __device__ __forceinline__ GemmRegion gemm_region_of_xcd(int tiles_m, int tiles_n, int xm, int xn, int xcd) {
    const int xr = xcd / xn, xc = xcd % xn;
    const int r_begin = (tiles_m * xr) / xm, r_end = (tiles_m * (xr + 1)) / xm;
    const int c_begin = (tiles_n * xc) / xn, c_end = (tiles_n * (xc + 1)) / xn;
    return GemmRegion{r_begin, c_begin, r_end - r_begin, c_end - c_begin};
}

// Tile (row, column) number `local` of a region in panel order; false past the end of the region.
__host__ __device__ __forceinline__ bool gemm_tile_of_region(const GemmRegion &reg, int local, int *tile_m, int *tile_n) {
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
    const GemmRegion reg = gemm_region_of_xcd(tiles_m, tiles_n, xm, xn, blockIdx.x & 7);  // workgroup b runs on XCD b % 8
    return gemm_tile_of_region(reg, blockIdx.x >> 3, tile_m, tile_n);
}

// ---- instruction-level helpers of the hand-scheduled GEMM loops --------------------------------------------------

// s_waitcnt immediate that waits until at most `n` vector-memory operations are outstanding and leaves the other
// counters alone (gfx9 encoding: vmcnt[3:0] in bits 3:0, vmcnt[5:4] in bits 15:14).
constexpr int waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

// LDS fragment read issued by hand so that it can be placed several MFMAs ahead of its use; the matching wait is
// tied to the destination registers, so nothing that consumes them can be scheduled above it.
template <int OFFSET>
__device__ __forceinline__ int4v_t lds_read_b128_early(uint32_t byte_addr) {
    int4v_t v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(byte_addr), "n"(OFFSET));
    return v;
}
// Wait until at most NEWER LDS reads issued after the one(s) that produce the given registers are outstanding.
template <int NEWER>
__device__ __forceinline__ void lds_wait_keep_newer(int4v_t &v) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(NEWER));
}
template <int NEWER>
__device__ __forceinline__ void lds_wait_keep_newer(int4v_t &lo, int4v_t &hi) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(lo), "+v"(hi) : "n"(NEWER));
}

// 16 bytes per lane from a buffer straight into LDS: lane i of the wave writes lds_dst + 16 * i (lds_dst must be
// wave-uniform), reading buffer offset voff (per lane) + soff (scalar).
__device__ __forceinline__ void buffer_load_to_lds_b128(__amdgpu_buffer_rsrc_t rsrc, uint4 *lds_dst, int voff, int soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void *)lds_dst, 16, voff, soff, 0, 0);
}

// Work item of this workgroup. The items of an XCD, in launch order: the tiles of its region that fill whole rounds
// of `concurrent` workgroups, then the remaining tiles cut into tail_parts K ranges each (tail_parts = 1: every tile
// is one item). `part` of `parts` is the K range, `slot` numbers the split tiles across the chip (fix-up storage).
struct GemmWorkItem {
    int tile_m, tile_n, part, parts, slot;
};

// (Workgroup `block` of the launch; a pure function so that the host can enumerate a launch, as the tests do.)
__host__ __device__ __forceinline__ bool gemm_work_item_of_block(int block, int tiles_m, int tiles_n, int xm, int xn,
                                                                 int concurrent, int tail_parts, int tail_stride,
                                                                 GemmWorkItem *item) {
    const GemmRegion reg = gemm_region_of_xcd(tiles_m, tiles_n, xm, xn, block & 7);
    const int region_tiles = reg.rows * reg.cols;
    const int whole = tail_parts > 1 ? (region_tiles / concurrent) * concurrent : region_tiles;
    int local = block >> 3;
    item->part = 0;
    item->parts = 1;
    item->slot = 0;
    if (local >= whole) {
        const int j = local - whole;
        local = whole + j / tail_parts;
        item->part = j % tail_parts;
        item->parts = tail_parts;
        item->slot = (block & 7) * tail_stride + j / tail_parts;
    }
    return gemm_tile_of_region(reg, local, &item->tile_m, &item->tile_n);
}

__device__ __forceinline__ bool gemm_work_item(int tiles_m, int tiles_n, int xm, int xn, int concurrent, int tail_parts,
                                               int tail_stride, GemmWorkItem *item) {
    return gemm_work_item_of_block(int(blockIdx.x), tiles_m, tiles_n, xm, xn, concurrent, tail_parts, tail_stride, item);
}

// Fix-up of a tile computed in K ranges by item.parts workgroups of THREADS threads, each holding R x T float4
// accumulators per thread. Every part writes its accumulators to the workspace (16 bytes per lane, agent scope),
// waits for the writes to be acknowledged and counts itself in; the part that arrives last reads all of them back
// in part order - so the sum does not depend on arrival order - and returns true with the sums in `acc`: it finishes
// the tile. The others return false. The counter goes back to zero for the next launch. `flag` is one int of LDS.
// Bit r of `rows_valid` says whether acc[r][*] holds rows inside the matrix: the others are exchanged at an offset
// past the end of the buffer, where the hardware drops stores and answers loads with zero without touching memory,
// which keeps the exchange of a short matrix (few valid rows in a tall tile) short. (Branching around them instead
// costs the GEMM kernels registers they do not have.)
template <int THREADS, int R, int T>
__device__ __forceinline__ bool gemm_k_split_fixup(float4_t (&acc)[R][T], const GemmWorkItem &item,
                                                   float *__restrict__ partials, uint32_t *__restrict__ counters, int *flag,
                                                   uint32_t rows_valid) {
    constexpr int kTileFloats = THREADS * R * T * 4;
    constexpr int kAgentScope = 1 << 4;  // sc1
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        partials + int64_t(item.slot) * item.parts * kTileFloats, 0, item.parts * kTileFloats * 4, 0x00020000);
    const int lane_off = threadIdx.x * 16;
    constexpr int kOutside = 0x7FFFFFF0;  // past the end of the buffer: the store is dropped, the load returns zero
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int off = ((rows_valid >> r) & 1u) ? lane_off : kOutside;
#pragma unroll
        for (int t = 0; t < T; ++t)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v_t, acc[r][t]), rsrc, off,
                                                   ((item.part * R + r) * T + t) * (THREADS * 16), kAgentScope);
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // vmcnt(0): every store of this lane has been acknowledged
    // The stores above write through (agent scope) and are complete; the fence tells the compiler, too, that nothing
    // may move across this point (at workgroup scope it emits no cache operation)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t old = __hip_atomic_fetch_add(&counters[item.slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = (old == uint32_t(item.parts - 1));
        if (*flag) __hip_atomic_store(&counters[item.slot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!*flag) return false;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // the reads below stay below (they bypass the L1 themselves)
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < T; ++t) acc[r][t] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int p = 0; p < item.parts; ++p) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int off = ((rows_valid >> r) & 1u) ? lane_off : kOutside;
            uint4v_t v[T];
#pragma unroll
            for (int t = 0; t < T; ++t)
                v[t] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, ((p * R + r) * T + t) * (THREADS * 16), kAgentScope);
#pragma unroll
            for (int t = 0; t < T; ++t) acc[r][t] += __builtin_bit_cast(float4_t, v[t]);
        }
    }
    return true;
}

// ---- runs across the tiles ------------------------------------------------------------------------------------------
//
// When an XCD has no whole number of rounds of tiles, equal K ranges per tile leave CUs idle (22 tiles on 32 CUs) or
// add rounds (66 thirds on 32 CUs). Here the (tile, stage) units of an XCD's region - tiles in panel order, a tile's
// stages in order - are cut into `wgs` runs of equal length, one per workgroup, whatever the tile boundaries: a
// workgroup computes the end of one tile, whole tiles, and the beginning of another. A bound closer than
// kGemmStreamMinStages to a tile boundary is moved onto it, so that no piece is shorter than a pipeline's prologue.
// A tile computed in pieces is summed by the workgroup that arrives last, in the order of the pieces
// (gemm_stream_fixup); its pieces come from consecutive workgroups, piece p from workgroup first + p. A workgroup
// leaves at most two pieces: the first of its run (kind 0) and, if that is a different one, the last (kind 1), which
// gives every piece a storage slot of its own, (workgroup, kind), however many tiles there are.
constexpr int kGemmStreamMinStages = 4;
constexpr int kGemmStreamMinShare = 4 * kGemmStreamMinStages;  // shortest run per workgroup the planner accepts: bounds stay apart

// First unit of workgroup j (0 .. wgs) of an XCD with `units` = tiles x stages units.
__host__ __device__ __forceinline__ int gemm_stream_bound(int units, int stages, int wgs, int j) {
    if (j <= 0) return 0;
    if (j >= wgs) return units;
    int raw = int((int64_t(units) * j) / wgs);
    const int t = raw / stages, r = raw - t * stages;
    if (r < kGemmStreamMinStages) raw = t * stages;
    else if (stages - r < kGemmStreamMinStages) raw = (t + 1) * stages;
    return raw;
}
// The workgroup whose run holds unit u.
__host__ __device__ __forceinline__ int gemm_stream_owner(int units, int stages, int wgs, int u) {
    int j = int((int64_t(u) * wgs) / units);  // moved bounds shift the answer by one at most
    while (j > 0 && gemm_stream_bound(units, stages, wgs, j) > u) --j;
    while (j + 1 < wgs && gemm_stream_bound(units, stages, wgs, j + 1) <= u) ++j;
    return j;
}

// One piece of a workgroup's run: stages [s_begin, s_end) of region tile `local`.
struct GemmStreamPiece {
    int local;           // tile of the XCD's region, in panel order
    int s_begin, s_end;
    int part, parts;     // parts == 1: the whole tile, nothing to exchange
    int first;           // workgroup (of the XCD) that computes piece 0
};
// Piece of workgroup j that lies in region tile `local` (the caller walks local from bound(j) / stages while
// local * stages < bound(j + 1)).
__host__ __device__ __forceinline__ GemmStreamPiece gemm_stream_piece(int units, int stages, int wgs, int j, int local) {
    const int lo = gemm_stream_bound(units, stages, wgs, j), hi = gemm_stream_bound(units, stages, wgs, j + 1);
    const int t0 = local * stages, t1 = t0 + stages;
    GemmStreamPiece p;
    p.local = local;
    p.s_begin = (lo > t0 ? lo : t0) - t0;
    p.s_end = (hi < t1 ? hi : t1) - t0;
    p.part = 0;
    p.parts = 1;
    p.first = j;
    if (p.s_begin != 0 || p.s_end != stages) {
        p.first = gemm_stream_owner(units, stages, wgs, t0);
        p.parts = gemm_stream_owner(units, stages, wgs, t1 - 1) - p.first + 1;
        p.part = j - p.first;
    }
    return p;
}
// Storage kind of the piece workgroup j holds of region tile `local`: 0 when the tile is the first of its run.
__host__ __device__ __forceinline__ int gemm_stream_kind(int units, int stages, int wgs, int j, int local) {
    return gemm_stream_bound(units, stages, wgs, j) / stages == local ? 0 : 1;
}

// Fix-up of a tile computed in pieces by runs across the tiles: as gemm_k_split_fixup, with every piece in its
// workgroup's own storage. `own` and `piece_at(p)` are the storage (THREADS * R * T * 4 floats each) of this
// workgroup's piece and of piece p of the tile, `counter` the tile's arrival counter (zero between launches).
template <int THREADS, int R, int T, typename PieceAt>
__device__ __forceinline__ bool gemm_stream_fixup(float4_t (&acc)[R][T], int parts, float *__restrict__ own, PieceAt piece_at,
                                                  uint32_t *__restrict__ counter, int *flag, uint32_t rows_valid) {
    constexpr int kTileFloats = THREADS * R * T * 4;
    constexpr int kAgentScope = 1 << 4;  // sc1
    constexpr int kOutside = 0x7FFFFFF0;  // past the end of the buffer: the store is dropped, the load returns zero
    const int lane_off = threadIdx.x * 16;
    {
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(own, 0, kTileFloats * 4, 0x00020000);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int off = ((rows_valid >> r) & 1u) ? lane_off : kOutside;
#pragma unroll
            for (int t = 0; t < T; ++t)
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v_t, acc[r][t]), rsrc, off, (r * T + t) * (THREADS * 16), kAgentScope);
        }
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // every store of this lane has been acknowledged (they write through)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t old = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = (old == uint32_t(parts - 1));
        if (*flag) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    const bool last = *flag != 0;
    __syncthreads();  // the flag is read by all before a later piece of this workgroup writes it again
    if (!last) return false;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < T; ++t) acc[r][t] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int p = 0; p < parts; ++p) {
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(piece_at(p), 0, kTileFloats * 4, 0x00020000);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int off = ((rows_valid >> r) & 1u) ? lane_off : kOutside;
            uint4v_t v[T];
#pragma unroll
            for (int t = 0; t < T; ++t) v[t] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, (r * T + t) * (THREADS * 16), kAgentScope);
#pragma unroll
            for (int t = 0; t < T; ++t) acc[r][t] += __builtin_bit_cast(float4_t, v[t]);
        }
    }
    return true;
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

// K ranges are worth their fix-up traffic only while an XCD has fewer tiles than `fill` workgroup slots: then as
// many parts (up to max_parts) as keep the busiest XCD within `fill`. For the int8 GEMM fill = 32, one workgroup per CU:
// a second co-resident workgroup buys nothing there (measured). The int4 GEMM spends more issue slots on
// dequantisation than on MFMAs, so a second workgroup per CU overlaps the two and fill = 64 pays. With whole rounds of
// workgroups in flight the kernels run at the chip's power limit and a shorter last round buys nothing (measured),
// so then the tail stays whole.
inline GemmTail make_gemm_tail(const GemmTiling &t, int concurrent, int fill, int max_parts) {
    GemmTail tail{1, 0, t.grid()};
    if (t.region_tiles >= concurrent || t.region_tiles == 0) return tail;
    for (int x = 0; x < 8; ++x) {
        const int n = gemm_region_tiles(t, x);
        if (n > tail.max_tiles) tail.max_tiles = n;
    }
    int parts = fill / t.region_tiles;
    if (parts > max_parts) parts = max_parts;
    tail.parts = parts < 1 ? 1 : parts;
    return tail;
}

// The same decision by counting rounds: with `concurrent` workgroup slots per XCD, the busiest XCD needs
// floor(n / concurrent) whole rounds plus ceil(rest * parts / concurrent) / parts of a round for its `rest` tail tiles
// cut into `parts` K ranges; the exchange of the partial tiles moves 8 * rest * parts tiles' worth of accumulators
// through memory, `exchange_cost` of a tile's compute time each (all workgroups share the memory system, so this adds
// up chip-wide). Takes the part count that minimises the sum if it saves at least a tenth of a round. Unlike
// make_gemm_tail this also splits a short tail behind whole rounds (33 tiles on 32 slots: 2 rounds -> 1.3), and does
// not split when that only trades one long round for several short ones of the same total (22 tiles on 32 slots: 2 or
// 3 parts change nothing, 4 parts save a quarter round but their exchange costs more than that).
inline GemmTail make_gemm_tail_by_rounds(const GemmTiling &t, int concurrent, int max_parts, double exchange_cost) {
    GemmTail tail{1, 0, t.grid()};
    int busiest = 0;
    for (int x = 0; x < 8; ++x) {
        const int n = gemm_region_tiles(t, x);
        if (n > busiest) busiest = n;
        if (n % concurrent > tail.max_tiles) tail.max_tiles = n % concurrent;
    }
    const int rest = busiest % concurrent;
    if (rest == 0) return tail;
    double best = 1.0;
    for (int p = 2; p <= max_parts; ++p) {
        const double rounds = double((rest * p + concurrent - 1) / concurrent) / p + 8.0 * rest * p * exchange_cost;
        if (rounds < best - 0.1) {
            best = rounds;
            tail.parts = p;
        }
    }
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
