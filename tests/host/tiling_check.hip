// Host-side enumeration of launches: every tile of the output must be computed exactly once (all of its K ranges or
// steps, each by one workgroup or wave), and GEMM tiles that are split must get distinct fix-up slots inside the planned storage.
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

// Runs across the tiles: every (tile, stage) of every XCD's region belongs to exactly one piece, a tile's pieces are
// numbered 0 .. parts - 1 in stage order and come from consecutive workgroups starting at `first`, no piece is shorter
// than kGemmStreamMinStages unless it is a whole tile's rest, and no two pieces share a storage slot (workgroup, kind).
static int check_stream(int tiles_m, int tiles_n, int stages, int wgs) {
    const GemmTiling t = make_gemm_tiling(tiles_m, tiles_n, wgs);
    std::vector<int> covered(size_t(tiles_m) * tiles_n * stages, 0);
    for (int xcd = 0; xcd < 8; ++xcd) {
        const GemmRegion reg = gemm_region_of_xcd(tiles_m, tiles_n, t.xm, t.xn, xcd);
        const int tiles = reg.rows * reg.cols, units = tiles * stages;
        if (tiles == 0) continue;
        if (int64_t(tiles) * stages < int64_t(wgs) * kGemmStreamMinShare) continue;  // the launcher does not use the plan then
        std::vector<int> parts_of(tiles, 0), next_part(tiles, 0), next_stage(tiles, 0), first_of(tiles, -1);
        std::vector<int> slot_used(size_t(wgs) * 2, 0);
        int prev = 0;
        for (int j = 0; j < wgs; ++j) {
            const int lo = gemm_stream_bound(units, stages, wgs, j), hi = gemm_stream_bound(units, stages, wgs, j + 1);
            if (lo != prev || hi <= lo) return std::printf("stream %dx%d s%d: workgroup %d of XCD %d runs [%d, %d) after %d\n", tiles_m, tiles_n, stages, j, xcd, lo, hi, prev), 1;
            prev = hi;
            for (int u = lo; u < hi; ++u)
                if (gemm_stream_owner(units, stages, wgs, u) != j) return std::printf("stream %dx%d s%d: owner of unit %d is not %d\n", tiles_m, tiles_n, stages, u, j), 1;
            int pieces = 0;
            for (int local = lo / stages; local * stages < hi; ++local) {
                const GemmStreamPiece p = gemm_stream_piece(units, stages, wgs, j, local);
                if (p.local != local || p.s_begin < 0 || p.s_end > stages || p.s_begin >= p.s_end || p.s_begin != next_stage[local])
                    return std::printf("stream %dx%d s%d: workgroup %d tile %d stages [%d, %d), expected from %d\n", tiles_m, tiles_n, stages, j, local, p.s_begin, p.s_end, next_stage[local]), 1;
                next_stage[local] = p.s_end;
                if (p.part != next_part[local] || (parts_of[local] != 0 && parts_of[local] != p.parts) || p.part >= p.parts ||
                    (first_of[local] >= 0 && first_of[local] != p.first) || p.first + p.part != j)
                    return std::printf("stream %dx%d s%d: workgroup %d tile %d part %d/%d first %d\n", tiles_m, tiles_n, stages, j, local, p.part, p.parts, p.first), 1;
                parts_of[local] = p.parts;
                first_of[local] = p.first;
                ++next_part[local];
                if (p.parts > 1) {
                    if (p.s_end - p.s_begin < kGemmStreamMinStages) return std::printf("stream %dx%d s%d: piece of %d stages\n", tiles_m, tiles_n, stages, p.s_end - p.s_begin), 1;
                    const int kind = gemm_stream_kind(units, stages, wgs, j, local);
                    if (slot_used[j * 2 + kind]++) return std::printf("stream %dx%d s%d: workgroup %d uses storage %d twice\n", tiles_m, tiles_n, stages, j, kind), 1;
                    ++pieces;
                } else if (p.s_begin != 0 || p.s_end != stages) {
                    return std::printf("stream %dx%d s%d: a lone piece [%d, %d)\n", tiles_m, tiles_n, stages, p.s_begin, p.s_end), 1;
                }
                int tm, tn;
                if (!gemm_tile_of_region(reg, local, &tm, &tn)) return std::printf("stream %dx%d: tile %d outside the region\n", tiles_m, tiles_n, local), 1;
                for (int st = p.s_begin; st < p.s_end; ++st) ++covered[(size_t(tm) * tiles_n + tn) * stages + st];
            }
            if (pieces > 2) return std::printf("stream %dx%d s%d: workgroup %d leaves %d pieces\n", tiles_m, tiles_n, stages, j, pieces), 1;
        }
        if (prev != units) return std::printf("stream %dx%d s%d: runs end at %d of %d\n", tiles_m, tiles_n, stages, prev, units), 1;
        for (int local = 0; local < tiles; ++local)
            if (next_stage[local] != stages || next_part[local] != parts_of[local])
                return std::printf("stream %dx%d s%d: tile %d ends at stage %d, %d of %d parts\n", tiles_m, tiles_n, stages, local, next_stage[local], next_part[local], parts_of[local]), 1;
    }
    for (int seen : covered)
        if (seen > 1) return std::printf("stream %dx%d s%d: a stage of a tile belongs to two XCDs\n", tiles_m, tiles_n, stages), 1;
    return 0;
}

// Bandwidth-bound kernels: the (tile, 32-row step) units of a launch are dealt to workgroups and waves in one flat run
// each. Every unit must belong to exactly one wave, a workgroup's run may touch two tiles at most, every tile has one
// collector (the workgroup with its last unit) that fetches exactly the slots of the workgroups before it in the tile,
// every other contributor sends exactly once into its own slot, and the plan never needs more mailbox than there is.
static int check_skinny(long long k, long long ncols, int hint, int rows, long long workspace_bytes, bool flat_ok, int cus) {
    static char dummy[16];
    const Workspace ws = split_workspace(dummy, workspace_bytes);
    if (workspace_bytes >= kCounterBytes &&
        (ws.mailbox_bytes < 0 || ws.mailbox_bytes > kMaxMailboxBytes || ws.mailbox_bytes % 256 != 0 ||
         kCounterBytes + ws.mailbox_bytes + ws.scratch_bytes != workspace_bytes ||
         reinterpret_cast<char *>(ws.mailbox) + ws.mailbox_bytes != ws.scratch))
        return std::printf("workspace of %lld bytes: mailbox %lld, scratch %lld\n", workspace_bytes, (long long)ws.mailbox_bytes, (long long)ws.scratch_bytes), 1;
    const SkinnyPlan free_plan = skinny_make_plan(k, ncols, hint, rows, 1LL << 40, true, flat_ok, cus);
    const bool fits = skinny_mailbox_need(free_plan, rows) <= ws.mailbox_bytes;
    bool threw = false;
    try {
        skinny_make_plan(k, ncols, hint, rows, ws.mailbox_bytes, true, flat_ok, cus);
    } catch (const Error &) { threw = true; }
    if (threw == fits) return std::printf("skinny k=%lld n=%lld rows=%d ws=%lld: strict error %d, fits %d\n", k, ncols, rows, workspace_bytes, threw, fits), 1;
    const SkinnyPlan p = skinny_make_plan(k, ncols, hint, rows, ws.mailbox_bytes, false, flat_ok, cus);
    if (fits && (p.groups != free_plan.groups)) return std::printf("skinny k=%lld n=%lld: a plan that fits was changed\n", k, ncols), 1;
    const int units = skinny_units(p);
    if (p.tiles != int((ncols + kSkinnyTileN - 1) / kSkinnyTileN) || p.ksteps != int((k + 31) / 32) || p.groups < p.tiles ||
        p.groups > units || p.groups > free_plan.groups || skinny_mailbox_need(p, rows) > ws.mailbox_bytes)
        return std::printf("skinny k=%lld n=%lld hint=%d rows=%d ws=%lld: %d tiles x %d steps, %d workgroups need %lld\n", k, ncols, hint, rows,
                           workspace_bytes, p.tiles, p.ksteps, p.groups, (long long)skinny_mailbox_need(p, rows)), 1;
    if (hint == 0 && p.groups > std::min(cus, 256) && p.groups != p.tiles)
        return std::printf("skinny k=%lld n=%lld: %d workgroups do not fit one round of %d CUs\n", k, ncols, p.groups, cus), 1;
    if (!flat_ok && p.splits == 0) return std::printf("skinny k=%lld n=%lld: runs across tiles where whole slices were asked for\n", k, ncols), 1;
    constexpr int kWaves = 8;
    std::vector<int> seen(units, 0), collector(p.tiles, -1), first(p.tiles, -1), sends(p.groups, 0), sent_to(p.groups, -1);
    int most = 0;
    // every run belongs to exactly one workgroup of the launch; with whole runs per tile a tile's runs share an XCD
    // (workgroup index mod 8) and are dispatched in run order
    std::vector<int> block_of(p.groups, -1);
    for (int b = 0; b < skinny_grid(p); ++b) {
        int g = -1;
        if (!skinny_group_of_block(p, p.tiles, b, &g)) continue;
        if (g < 0 || g >= p.groups || block_of[g] >= 0) return std::printf("skinny k=%lld n=%lld: workgroup %d -> run %d\n", k, ncols, b, g), 1;
        block_of[g] = b;
    }
    for (int g = 0; g < p.groups; ++g) {
        if (block_of[g] < 0) return std::printf("skinny k=%lld n=%lld: run %d has no workgroup\n", k, ncols, g), 1;
        if (p.splits > 0 && g % p.splits != 0 && (block_of[g] % 8 != block_of[g - 1] % 8 || block_of[g] < block_of[g - 1]))
            return std::printf("skinny k=%lld n=%lld: runs %d and %d of one tile on workgroups %d and %d\n", k, ncols, g - 1, g, block_of[g - 1], block_of[g]), 1;
    }
    if (p.splits > 0 && p.groups != p.tiles * p.splits) return std::printf("skinny k=%lld n=%lld: %d splits, %d runs, %d tiles\n", k, ncols, p.splits, p.groups, p.tiles), 1;
    for (int g = 0; g < p.groups; ++g) {
        const SkinnyWork wk = skinny_work_of(p, g);
        if (p.splits > 0 && (wk.crosses() || wk.tile != g / p.splits)) return std::printf("skinny k=%lld n=%lld: run %d of %d per tile crosses out of tile %d\n", k, ncols, g, p.splits, wk.tile), 1;
        if (wk.u0 != skinny_first_unit(p, g) || wk.u1 <= wk.u0 || wk.u1 > units || wk.tile != wk.u0 / p.ksteps ||
            (wk.u1 - 1) / p.ksteps > wk.tile + 1 || skinny_group_of_unit(p, wk.u0) != g || skinny_group_of_unit(p, wk.u1 - 1) != g)
            return std::printf("skinny k=%lld n=%lld: workgroup %d runs [%d, %d) from tile %d\n", k, ncols, g, wk.u0, wk.u1, wk.tile), 1;
        const SkinnyRoles roles = skinny_roles_of(p, wk, g, kWaves);
        int at = wk.u0;
        for (int wv = 0; wv < kWaves; ++wv) {
            int lo, hi, part;
            skinny_wave_run(wk, wv, kWaves, &lo, &hi, &part);
            if (lo != at || hi < lo) return std::printf("skinny k=%lld n=%lld: workgroup %d wave %d runs [%d, %d), expected from %d\n", k, ncols, g, wv, lo, hi, at), 1;
            // a wave's run lies in one tile, and its LDS slot (= its index) is one of that tile's
            if (part != (wv >= roles.c0) || (part == 0 && hi > wk.bound) || (part == 1 && (lo < wk.bound || !wk.crosses())))
                return std::printf("skinny k=%lld n=%lld: workgroup %d wave %d runs [%d, %d) for part %d, boundary at %d, %d waves before it\n", k, ncols, g, wv, lo, hi, part, wk.bound, roles.c0), 1;
            if (hi - lo > (wk.u1 - wk.u0 + kWaves - 2) / (kWaves - 1) + 1)  // two groups of waves: no wave beyond a seventh of the run (and rounding)
                return std::printf("skinny k=%lld n=%lld: workgroup %d wave %d has %d of %d steps\n", k, ncols, g, wv, hi - lo, wk.u1 - wk.u0), 1;
            for (int u = lo; u < hi; ++u) ++seen[u];
            at = hi;
        }
        if (at != wk.u1) return std::printf("skinny k=%lld n=%lld: workgroup %d waves end at %d, run at %d\n", k, ncols, g, at, wk.u1), 1;
        if (roles.c0 < 1 || roles.c0 > kWaves || (wk.crosses() && roles.c0 == kWaves))
            return std::printf("skinny k=%lld n=%lld: workgroup %d: %d waves before the boundary\n", k, ncols, g, roles.c0), 1;
        // roles
        if (first[wk.tile] < 0) first[wk.tile] = g;
        if (roles.finish != int(wk.collects()) || (roles.send_slot >= 0) != (wk.crosses() || !wk.collects()) || (roles.send_slot >= 0 && roles.send_slot != g) ||
            roles.send_tile != (wk.crosses() ? wk.tile + 1 : wk.tile) ||
            (roles.send_slot >= 0 && (roles.send_lo != (wk.crosses() ? roles.c0 : 0) || roles.send_hi != kWaves)))
            return std::printf("skinny k=%lld n=%lld: workgroup %d: finish %d, sends LDS slots [%d, %d) to slot %d for tile %d\n", k, ncols, g, roles.finish, roles.send_lo, roles.send_hi,
                               roles.send_slot, roles.send_tile), 1;
        if (wk.collects()) {
            if (collector[wk.tile] >= 0) return std::printf("skinny k=%lld n=%lld: tile %d has two collectors\n", k, ncols, wk.tile), 1;
            collector[wk.tile] = g;
            if (roles.fetch_first != first[wk.tile] || roles.fetch_others != g - first[wk.tile])
                return std::printf("skinny k=%lld n=%lld: workgroup %d fetches %d slots from %d, the tile's first is %d\n", k, ncols, g, roles.fetch_others, roles.fetch_first, first[wk.tile]), 1;
            most = std::max(most, roles.fetch_others);
        } else {
            ++sends[g];
            sent_to[g] = wk.tile;
        }
        if (wk.crosses()) {
            if (wk.tile + 1 >= p.tiles || first[wk.tile + 1] >= 0) return std::printf("skinny k=%lld n=%lld: workgroup %d crosses into a tile that has begun\n", k, ncols, g), 1;
            first[wk.tile + 1] = g;
            ++sends[g];
            sent_to[g] = wk.tile + 1;
        } else if (wk.collects() && wk.tile + 1 < p.tiles && skinny_first_unit(p, g + 1) != wk.bound) {
            return std::printf("skinny k=%lld n=%lld: workgroup %d ends at a tile boundary that the next does not start at\n", k, ncols, g), 1;
        }
    }
    for (int u = 0; u < units; ++u)
        if (seen[u] != 1) return std::printf("skinny k=%lld n=%lld: unit %d belongs to %d waves\n", k, ncols, u, seen[u]), 1;
    for (int t = 0; t < p.tiles; ++t) {
        if (collector[t] < 0 || first[t] < 0 || first[t] > collector[t]) return std::printf("skinny k=%lld n=%lld: tile %d has no collector\n", k, ncols, t), 1;
        for (int g = first[t]; g < collector[t]; ++g)
            if (sends[g] != 1 || sent_to[g] != t) return std::printf("skinny k=%lld n=%lld: workgroup %d should send once to tile %d\n", k, ncols, g, t), 1;
    }
    for (int g = 0; g < p.groups; ++g)
        if (sends[g] > 1) return std::printf("skinny k=%lld n=%lld: workgroup %d sends twice\n", k, ncols, g), 1;
    if (most != p.max_others) return std::printf("skinny k=%lld n=%lld: max_others %d, enumerated %d\n", k, ncols, p.max_others, most), 1;
    if ((p.groups == p.tiles) != (most == 0)) return std::printf("skinny k=%lld n=%lld: %d workgroups, %d tiles, %d partial tiles fetched\n", k, ncols, p.groups, p.tiles, most), 1;
    return 0;
}

int main() {
    long long n = 0;
    // 16384 x 128256 with 8 rows (an lm_head decode batch) has 501 tiles: one workgroup each, nothing exchanged; small
    // workspaces cut a plan down to what their mailbox holds
    for (long long ws : {0LL, 1024LL, 65536LL, 65536LL + 8192, 1LL << 20, 16LL << 20, (16LL << 20) + 65536, 64LL << 20, 96LL << 20})
        for (long long k : {32LL, 96LL, 128LL, 1000LL, 4096LL, 11008LL, 16384LL, 28672LL})
            for (long long nc : {2LL, 16LL, 256LL, 272LL, 4096LL, 11008LL, 12288LL, 128256LL})
                for (int rows : {1, 2, 8, 16})
                    for (int hint : {0, 1, 3, 8, 64}) {
                        if (check_skinny(k, nc, hint, rows, ws, true, 256)) return 1;
                        if (check_skinny(k, nc, hint, rows, ws, false, 256)) return 1;
                        n += 2;
                        // fewer CUs than a full device (a partition), more than the plan's cap
                        if (hint == 0 && (ws == 0 || ws == (64LL << 20))) {
                            for (int cus : {1, 32, 64, 80, 304})
                                if (check_skinny(k, nc, hint, rows, ws, rows == 1, cus)) return 1;
                            n += 5;
                        }
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
    for (int stages : {16, 17, 43, 64, 172, 448})
        for (int tm = 1; tm <= 40; tm += (tm < 10 ? 1 : 5))
            for (int tn = 1; tn <= 130; tn += (tn < 50 ? 3 : 9))
                for (int wgs : {32, 64}) {
                    if (check_stream(tm, tn, stages, wgs)) return 1;
                    ++n;
                }
    std::printf("ok %lld launches\n", n);
    return 0;
}
