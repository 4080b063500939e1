// Host-side enumeration of launches: every tile of the output must be computed exactly once (all of its K ranges or
// slices, each by one workgroup), and GEMM tiles that are split must get distinct fix-up slots inside the planned storage.
// Built and run by tests/test_tiling.py; exits non-zero with a message on the first violation.
#include <cstdio>
#include <vector>

#include "gemm_tiling.h"
#include "skinny_common.h"

using namespace qmm;

// mode 0: the planner by fill; 1: no K ranges; 2: the planner by rounds (fill = the exchange cost in 1e-4 of a tile's time);
// 3: as 2 with the regions laid out for twice as many workgroups at a time as the rounds are counted in (two per CU)
static int check(int tiles_m, int tiles_n, int concurrent, int fill, int max_parts, int mode) {
    const GemmTiling t = make_gemm_tiling(tiles_m, tiles_n, mode == 3 ? 2 * concurrent : concurrent);
    if (t.xm * t.xn != 8) return std::printf("tiling %dx%d: %d x %d regions\n", tiles_m, tiles_n, t.xm, t.xn), 1;
    GemmTail tail = make_gemm_tail(t, concurrent, fill, max_parts);
    if (mode == 1) tail = GemmTail{1, 0, t.grid()};
    if (mode >= 2) {
        tail = make_gemm_tail_by_rounds(t, concurrent, max_parts, fill * 1e-4);
        if (tail.parts < 1 || tail.parts > max_parts || tail.max_tiles >= concurrent)
            return std::printf("%dx%d c%d: plan by rounds gives %d parts, %d tail tiles\n", tiles_m, tiles_n, concurrent, tail.parts, tail.max_tiles), 1;
    }
    const long long grid = gemm_grid_with_tail(t, concurrent, tail);
    std::vector<int> seen(size_t(tiles_m) * tiles_n * max_parts, 0), parts_of(size_t(tiles_m) * tiles_n, 0);
    std::vector<int> slot_owner(size_t(8) * (tail.max_tiles > 0 ? tail.max_tiles : 1), -1);
    for (long long b = 0; b < grid; ++b) {
        GemmWorkItem it;
        if (!gemm_work_item_of_block(int(b), tiles_m, tiles_n, t.xm, t.xn, concurrent, tail.parts, tail.max_tiles, &it)) continue;
        if (it.tile_m < 0 || it.tile_m >= tiles_m || it.tile_n < 0 || it.tile_n >= tiles_n || it.part < 0 || it.part >= it.parts ||
            it.parts > max_parts)
            return std::printf("%dx%d c%d: block %lld -> tile (%d, %d) part %d/%d\n", tiles_m, tiles_n, concurrent, b, it.tile_m,
                               it.tile_n, it.part, it.parts), 1;
        const size_t tile = size_t(it.tile_m) * tiles_n + it.tile_n;
        if (parts_of[tile] != 0 && parts_of[tile] != it.parts)
            return std::printf("%dx%d c%d: tile %zu seen with %d and %d parts\n", tiles_m, tiles_n, concurrent, tile, parts_of[tile], it.parts), 1;
        parts_of[tile] = it.parts;
        if (seen[tile * max_parts + it.part]++)
            return std::printf("%dx%d c%d: tile %zu part %d computed twice\n", tiles_m, tiles_n, concurrent, tile, it.part), 1;
        if (it.parts > 1) {
            if (it.slot < 0 || it.slot >= int(slot_owner.size()))
                return std::printf("%dx%d c%d: slot %d outside %zu\n", tiles_m, tiles_n, concurrent, it.slot, slot_owner.size()), 1;
            if (slot_owner[it.slot] >= 0 && slot_owner[it.slot] != int(tile))
                return std::printf("%dx%d c%d: slot %d shared by tiles %d and %zu\n", tiles_m, tiles_n, concurrent, it.slot, slot_owner[it.slot], tile), 1;
            slot_owner[it.slot] = int(tile);
        }
    }
    for (size_t tile = 0; tile < parts_of.size(); ++tile) {
        if (parts_of[tile] == 0) return std::printf("%dx%d c%d: tile %zu never computed\n", tiles_m, tiles_n, concurrent, tile), 1;
        for (int p = 0; p < parts_of[tile]; ++p)
            if (seen[tile * max_parts + p] != 1)
                return std::printf("%dx%d c%d: tile %zu part %d missing\n", tiles_m, tiles_n, concurrent, tile, p), 1;
    }
    return 0;
}

// Bandwidth-bound kernels: K is cut into `splits` slices of rows_per_block rows (whole multiples of the granule) that
// cover K exactly once, and every (column tile, slice) pair belongs to exactly one workgroup.
static int check_skinny(long long k, long long ncols, int slice_rows, int hint, int granule) {
    int rpb = 0, splits = 0, tiles = 0;
    if (slice_rows > 0) skinny_plan(k, ncols, slice_rows, hint, granule, &rpb, &splits, &tiles);
    else skinny_plan_one_round(k, ncols, granule / 32, hint, &rpb, &splits, &tiles);  // the int8 kernel's plan
    if (slice_rows == 0 && hint == 0 && (long long)(splits) * tiles > 256 && splits > 1)
        return std::printf("skinny k=%lld n=%lld: %d slices x %d tiles do not fit one round\n", k, ncols, splits, tiles), 1;
    if (rpb <= 0 || rpb % granule != 0 || splits < 1 || (long long)(splits) * rpb < k || (long long)(splits - 1) * rpb >= k ||
        tiles != int((ncols + kSkinnyTileN - 1) / kSkinnyTileN))
        return std::printf("skinny k=%lld n=%lld hint=%d: rows %d x %d splits, %d tiles\n", k, ncols, hint, rpb, splits, tiles), 1;
    std::vector<int> seen(size_t(tiles) * splits, 0);
    const int grid = ((tiles + 7) / 8) * 8 * splits;
    for (int b = 0; b < grid; ++b) {
        int tile, split;
        if (!skinny_tile_of(b, splits, tiles, &tile, &split)) continue;
        if (tile < 0 || split < 0 || split >= splits || seen[size_t(tile) * splits + split]++)
            return std::printf("skinny k=%lld n=%lld: block %d -> tile %d split %d\n", k, ncols, b, tile, split), 1;
    }
    for (int v : seen)
        if (v != 1) return std::printf("skinny k=%lld n=%lld: a slice has no workgroup\n", k, ncols), 1;
    return 0;
}

// A plan cut down to a mailbox: still whole granules covering K once, never more bytes than the mailbox holds, the
// plan untouched when it fits, and a strict caller gets an error exactly when it does not.
static int check_fit(long long k, long long ncols, int rows, long long workspace_bytes, int granule) {
    int rpb = 0, splits = 0, tiles = 0;
    if (granule == 256) skinny_plan_one_round(k, ncols, 8, 0, &rpb, &splits, &tiles);
    else skinny_plan(k, ncols, rows > 8 ? 768 : 512, 0, granule, &rpb, &splits, &tiles);
    const int rpb0 = rpb, splits0 = splits;
    static char dummy[16];
    const Workspace ws = split_workspace(dummy, workspace_bytes);
    if (workspace_bytes >= kCounterBytes &&
        (ws.mailbox_bytes < 0 || ws.mailbox_bytes > kMaxMailboxBytes || ws.mailbox_bytes % 256 != 0 ||
         kCounterBytes + ws.mailbox_bytes + ws.scratch_bytes != workspace_bytes ||
         reinterpret_cast<char *>(ws.mailbox) + ws.mailbox_bytes != ws.scratch))
        return std::printf("workspace of %lld bytes: mailbox %lld, scratch %lld\n", workspace_bytes, (long long)ws.mailbox_bytes, (long long)ws.scratch_bytes), 1;
    const bool fits = skinny_mailbox_need(tiles, splits, rows) <= ws.mailbox_bytes;
    bool threw = false;
    try {
        int r2 = rpb, s2 = splits;
        skinny_fit_mailbox(k, granule, tiles, rows, ws.mailbox_bytes, true, &r2, &s2);
    } catch (const Error &) { threw = true; }
    if (threw == fits) return std::printf("fit k=%lld n=%lld rows=%d ws=%lld: strict error %d, fits %d\n", k, ncols, rows, workspace_bytes, threw, fits), 1;
    skinny_fit_mailbox(k, granule, tiles, rows, ws.mailbox_bytes, false, &rpb, &splits);
    if (fits && (rpb != rpb0 || splits != splits0)) return std::printf("fit k=%lld n=%lld: a plan that fits was changed\n", k, ncols), 1;
    if (rpb <= 0 || rpb % granule != 0 || splits < 1 || splits > splits0 || (long long)(splits) * rpb < k || (long long)(splits - 1) * rpb >= k ||
        skinny_mailbox_need(tiles, splits, rows) > ws.mailbox_bytes)
        return std::printf("fit k=%lld n=%lld rows=%d ws=%lld: rows %d x %d splits need %lld\n", k, ncols, rows, workspace_bytes, rpb, splits,
                           (long long)skinny_mailbox_need(tiles, splits, rows)), 1;
    return 0;
}

int main() {
    long long n = 0;
    // 16384 x 128256 with 8 rows (an lm_head decode batch) wants 131 MB of partial tiles: it must come out within the mailbox
    for (long long ws : {0LL, 1024LL, 65536LL, 65536LL + 8192, 1LL << 20, 16LL << 20, (16LL << 20) + 65536, 64LL << 20, 96LL << 20})
        for (long long k : {128LL, 4096LL, 11008LL, 16384LL})
            for (long long nc : {256LL, 4096LL, 11008LL, 128256LL})
                for (int rows : {1, 8, 16})
                    for (int granule : {128, 256, 512}) {
                        if (check_fit(k, nc, rows, ws, granule)) return 1;
                        ++n;
                    }
    for (long long k : {32LL, 96LL, 128LL, 1000LL, 4096LL, 11008LL, 8192LL, 28672LL})
        for (long long nc : {2LL, 16LL, 256LL, 272LL, 4096LL, 11008LL, 12288LL})
            for (int hint : {0, 1, 3, 8, 64})
                for (int cfg = 0; cfg < 5; ++cfg) {
                    if (check_skinny(k, nc, cfg == 1 ? 768 : cfg >= 3 ? 0 : 512, hint, cfg == 2 || cfg == 3 ? 256 : 128)) return 1;
                    ++n;
                }
    const int cfgs[][3] = {{32, 32, 4}, {32, 32, 8}, {64, 64, 4}, {64, 32, 4}};  // concurrent, fill, max_parts of the launchers
    for (const auto &c : cfgs)
        for (int tm = 1; tm <= 70; tm += (tm < 20 ? 1 : 7))
            for (int tn = 1; tn <= 130; tn += (tn < 50 ? 1 : 9)) {
                if (check(tm, tn, c[0], c[1], c[2], 0)) return 1;
                if (check(tm, tn, c[0], c[1], c[2], 1)) return 1;
                if (check(tm, tn, c[0], 7, c[2], 2)) return 1;
                if (check(tm, tn, c[0], 0, c[2], 2)) return 1;  // free exchange: splits wherever a round is partly filled
                if (check(tm, tn, c[0], 2, c[2], 3)) return 1;
                n += 5;
            }
    std::printf("ok %lld launches\n", n);
    return 0;
}
