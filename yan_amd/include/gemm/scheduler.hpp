// Workgroup -> output-tile mapping for a 256-CU, 8-XCD part.
// Replaces the reference's persistent tile Scheduler (yan/include/gemm/scheduler.cuh:15-58: block count
// ceil(m/BLOCK_M)*ceil(N/BLOCK_N), grouped swizzle of 16 blocks for L2 reuse). The mapping is the same for all
// three GemmTypes; what a group changes (operand bases, valid rows) is applied by the kernel on top of the tile.
#pragma once

#include "utils.hpp"

namespace yan {

enum class GemmType { Normal, GroupedContiguous, GroupedMasked };

struct TileCoord {
    int  m_idx;
    int  n_idx;
    bool valid;
};

// The hardware hands consecutive workgroup ids to the 8 XCDs round-robin, and each XCD has a private L2.
// Workgroup `bid` therefore runs on XCD `bid % 8`, and the 32 tiles an XCD has in flight should form a compact
// GROUP_M x 4 patch whose A and B panels are shared through that L2. Two arrangements do that; both have the same
// number of slots and give every XCD the same number of tiles.
//
// Band order (the default): every XCD gets one contiguous range of a tile sequence that walks bands of GROUP_M
// tile-rows column by column.
//
// Region order (chosen when the operands together do not fit the 256 MB memory-side cache; the caller passes
// `row_bytes`, the bytes of one operand row = K * element size): the 8 patches that run at the
// same time form one region of R x (256 / R) tiles, R = 16, 32, 8 or 64, and the regions are walked along one dimension
// first, so that the panels of the other dimension stay in the cache while those of the first stream through. Band
// order keeps up to 8 x 8 + 4 x 8 different panels in flight chip-wide and re-reads a whole operand from HBM for every
// round once they outgrow the cache; here the region shape and the direction are the ones a small traffic model rates
// cheapest (ties go to the squarer region). Measured on bf16 with 256 x 256 tiles: 12288^3 3067 -> 2737 us,
// 8192 x 4096 x 14336 735 -> 683, 16384^2 x 8192 3195 -> 2995; no change where the model picks what band order amounts
// to (8192^2 x 12288). FP8: 16384^3 3627 -> 3506 us.
template <int GROUP_M = 8>
struct XcdTileScheduler {
    static constexpr int PATCH_COLS = 4, PATCH = GROUP_M * PATCH_COLS, ROUND = PATCH * kNumXCD;
    static constexpr long long kCacheBytes = 256ll << 20;

    int  tiles_m, tiles_n, total, per_xcd;
    int  band_height;                     // tile-rows of a band: GROUP_M, or fewer when the caller's groups hold fewer (below)
    int  region_rows, region_cols;        // 0: band order
    bool rows_outer;                      // region order: all column blocks of a row block before the next row block

    __host__ __device__ XcdTileScheduler(int m, int n, int block_m, int block_n, long long row_bytes = 0) {
        tiles_m = ceil_div(m, block_m);
        tiles_n = ceil_div(n, block_n);
        total   = tiles_m * tiles_n;
        per_xcd = ceil_div(total, kNumXCD);
        band_height = GROUP_M;
        region_rows = region_cols = 0;
        rows_outer = true;
        const long long panel_a = row_bytes * block_m, panel_b = row_bytes * block_n;
        const long long all_a = panel_a * tiles_m, all_b = panel_b * tiles_n;
        if (row_bytes <= 0 || total < ROUND || all_a + all_b <= kCacheBytes) return;
        long long best = -1;
        static_assert(GROUP_M == 8 && ROUND == 256);
        const int candidates[4] = {16, 32, 8, 64};          // region rows; ties go to the earlier (squarer) one
        for (int i = 0; i < 4; ++i) {
            const int r = candidates[i], c = ROUND / r;
            if (r > ceil_div(tiles_m, GROUP_M) * GROUP_M || c > ceil_div(tiles_n, PATCH_COLS) * PATCH_COLS) continue;
            const int re = r < tiles_m ? r : tiles_m, ce = c < tiles_n ? c : tiles_n;
            const int row_blocks = ceil_div(tiles_m, r), col_blocks = ceil_div(tiles_n, c);
            const bool block_fits = re * panel_a + ce * panel_b <= kCacheBytes;
            // rows outer: the A block stays while the column blocks pass; B is read once per row block unless all of it stays
            const long long a_outer = (block_fits ? all_a : all_a * col_blocks) +
                                      ((col_blocks == 1 && all_b + re * panel_a <= kCacheBytes) ? all_b : all_b * row_blocks);
            const long long b_outer = (block_fits ? all_b : all_b * row_blocks) +
                                      ((row_blocks == 1 && all_a + ce * panel_b <= kCacheBytes) ? all_a : all_a * col_blocks);
            if (best < 0 || a_outer < best) { best = a_outer; region_rows = r; region_cols = c; rows_outer = true; }
            if (b_outer < best)             { best = b_outer; region_rows = r; region_cols = c; rows_outer = false; }
        }
    }

    __host__ __device__ int grid_size() const { return per_xcd * kNumXCD; }

    __host__ __device__ TileCoord tile_of(int bid) const {
        if (region_rows) return region_tile_of(bid);
        const int t = (bid % kNumXCD) * per_xcd + bid / kNumXCD;
        if (t >= total) return {0, 0, false};
        return band_tile(t);
    }

    // Grouped layouts: the rows are `groups` stacked problems with their own weights. Bands no taller than a group keep the
    // 32 consecutive tiles an XCD runs at once inside one group where groups are aligned: h x (32 / h) tiles share h
    // activation panels and 32 / h weight panels of one group, instead of 8 and 4 per group touched (4 groups of 4 tile-rows:
    // 12 panels instead of 16).
    __host__ __device__ void fit_bands_to_groups(int tile_rows_per_group) {
        band_height = tile_rows_per_group < 1 ? 1 : (tile_rows_per_group < GROUP_M ? tile_rows_per_group : GROUP_M);
    }

    // Tile number t of the band-order sequence.
    __host__ __device__ TileCoord band_tile(int t) const {
        const int band      = band_height * tiles_n;
        const int first_m   = (t / band) * band_height;
        const int band_rows = (tiles_m - first_m) < band_height ? (tiles_m - first_m) : band_height;
        const int in_band   = t % band;
        return {first_m + in_band % band_rows, in_band / band_rows, true};
    }

    // Slot -> position in a tile sequence, dealt out in rounds: full rounds of 256 tiles hand XCD x the x-th run of 32
    // consecutive tiles; the tiles left after the full rounds are dealt out in 8 equal runs. -1: an empty slot.
    __host__ __device__ int dealt_position(int bid) const {
        const int x = bid % kNumXCD, q = bid / kNumXCD;
        const int full = total / ROUND, rest = total - full * ROUND;
        if (q < full * PATCH) return ((q / PATCH) * kNumXCD + x) * PATCH + q % PATCH;
        const int run = ceil_div(rest, kNumXCD), q_rest = q - full * PATCH;
        const int t = full * ROUND + x * run + q_rest;
        return (q_rest >= run || t >= total) ? -1 : t;
    }

    // Band order dealt out in rounds: an XCD's 32 concurrent tiles are still a patch of one band, but consecutive patches
    // go to different XCDs. For grids whose tiles differ in cost by position (the masked layout: a group may have few rows
    // or none), where a contiguous range per XCD would leave some XCDs with all the work.
    __host__ __device__ TileCoord dealt_band_tile_of(int bid) const {
        const int t = dealt_position(bid);
        if (t < 0) return {0, 0, false};
        return band_tile(t);
    }

    // Region order, dealt out in rounds (a run of 32 consecutive tiles is one patch when the region is whole). The sequence: region
    // by region; inside a region patch rows of GROUP_M, inside a patch row patches of 4 columns, inside a patch column by
    // column. Regions, patch rows and patches at the lower and right edges are smaller, which shifts the runs against
    // the patches but loses no tile.
    __host__ __device__ TileCoord region_tile_of(int bid) const {
        const int t = dealt_position(bid);
        if (t < 0) return {0, 0, false};
        int rb, cb, hh, ww, p;        // region (rb, cb) of hh x ww tiles, position p inside it
        if (rows_outer) {
            rb = t / (region_rows * tiles_n);
            hh = (tiles_m - rb * region_rows) < region_rows ? (tiles_m - rb * region_rows) : region_rows;
            const int in_block = t - rb * region_rows * tiles_n;
            cb = in_block / (hh * region_cols);
            ww = (tiles_n - cb * region_cols) < region_cols ? (tiles_n - cb * region_cols) : region_cols;
            p  = in_block - cb * hh * region_cols;
        } else {
            cb = t / (region_cols * tiles_m);
            ww = (tiles_n - cb * region_cols) < region_cols ? (tiles_n - cb * region_cols) : region_cols;
            const int in_block = t - cb * region_cols * tiles_m;
            rb = in_block / (ww * region_rows);
            hh = (tiles_m - rb * region_rows) < region_rows ? (tiles_m - rb * region_rows) : region_rows;
            p  = in_block - rb * ww * region_rows;
        }
        const int pr = p / (GROUP_M * ww);                                       // patch row
        const int ph = (hh - pr * GROUP_M) < GROUP_M ? (hh - pr * GROUP_M) : GROUP_M;
        const int in_row = p - pr * GROUP_M * ww;
        const int pc = in_row / (ph * PATCH_COLS);                               // patch
        const int in_patch = in_row - pc * ph * PATCH_COLS;
        return {rb * region_rows + pr * GROUP_M + in_patch % ph, cb * region_cols + pc * PATCH_COLS + in_patch / ph, true};
    }
};

// Slot numbering of the masked layout. Only the first masked_m[g] rows of a group exist, and the caller's `expected_m`
// says how many that usually is: the tile rows below it come first, all groups' stacked along m into one grid whose
// patches of 32 tiles (8 x 4, or as tall as a group where groups hold fewer tile-rows) are dealt out to the XCDs in turn (the
// 32 tiles an XCD runs at once share weight panels through its L2; consecutive patches go to different XCDs, so a group with few rows or none does not
// leave one XCD idle), the tile rows above it afterwards in a second grid of the same kind. A workgroup whose tile does not exist leaves at once, but
// it still takes a compute unit to start: numbered group by group, existing and empty tiles alternate and the existing
// ones start in ever smaller waves as the empty ones get out of their way (8 groups x 128 rows of which 64 exist: 58 us
// against 42 us when the rows are 64). Same on the host (slot count) and on the device (slot -> group, tile).
struct MaskedSlots {
    XcdTileScheduler<> likely, rest;
    int tiles_m, likely_rows, likely_slots;

    __host__ __device__ MaskedSlots(int num_groups, int m, int n, int block_m, int block_n, int expected_m)
        : likely(0, 0, block_m, block_n), rest(0, 0, block_m, block_n) {
        tiles_m = ceil_div(m, block_m);
        likely_rows = expected_m > 0 ? ceil_div(expected_m, block_m) : tiles_m;
        likely_rows = likely_rows < tiles_m ? likely_rows : tiles_m;
        likely = XcdTileScheduler<>(num_groups * likely_rows * block_m, n, block_m, block_n);
        rest   = XcdTileScheduler<>(num_groups * (tiles_m - likely_rows) * block_m, n, block_m, block_n);
        likely.fit_bands_to_groups(likely_rows);
        rest.fit_bands_to_groups(tiles_m - likely_rows);
        likely_slots = likely.grid_size();
    }

    __host__ __device__ long long num_slots() const { return (long long)likely_slots + rest.grid_size(); }

    // group and tile (within the group's [m, n] problem) of a slot
    __host__ __device__ TileCoord tile_of(int slot, int* group) const {
        const bool first = slot < likely_slots;
        const int rows = first ? likely_rows : tiles_m - likely_rows;
        TileCoord t = first ? likely.dealt_band_tile_of(slot) : rest.dealt_band_tile_of(slot - likely_slots);
        if (!t.valid) { *group = 0; return t; }
        *group = t.m_idx / rows;
        t.m_idx = t.m_idx % rows + (first ? 0 : likely_rows);
        return t;
    }
};

// Slot numbering of the contiguous layout on 256-row tiles. A tile row whose two 128-row halves belong to two groups makes
// two passes over K and takes about half as long again as the others; started last, one of them ends alone after everyone
// else. `two_group_rows` of the `tiles_m` rows are of that kind (the kernel counts them in the caller's layout; the host
// does not know them and launches `num_slots()` workgroups whatever their number). Their tiles come first in every XCD's
// share of the slots and are dealt to the XCDs one by one, so that every XCD gets as many (an XCD runs its own slots, and
// a patch of 32 slow tiles would fall to one of them); the other rows follow in band order dealt out in patches of 32.
// `tile_of` names rows by position: positions below `two_group_rows` are the two-group rows, the others follow, either
// kind in ascending order. With no such row the order is the plain one (a contiguous range of the band order per XCD).
struct ContiguousSlots {
    XcdTileScheduler<> all, rest;
    int two_group_rows, first_tiles;

    __host__ __device__ ContiguousSlots(int m, int n, int block_m, int block_n, int num_groups, int two_group_rows_)
        : all(m, n, block_m, block_n), rest(0, 0, block_m, block_n), two_group_rows(two_group_rows_) {
        all.fit_bands_to_groups(all.tiles_m / (num_groups > 0 ? num_groups : 1));
        rest = XcdTileScheduler<>((all.tiles_m - two_group_rows) * block_m, n, block_m, block_n);
        rest.band_height = all.band_height;
        first_tiles = two_group_rows * all.tiles_n;
    }

    // one slot per XCD more than the tiles need: the two kinds of rows are rounded up to whole slots per XCD separately
    __host__ __device__ static long long num_slots(int m, int n, int block_m, int block_n) {
        return (long long)XcdTileScheduler<>(m, n, block_m, block_n).grid_size() + kNumXCD;
    }

    __host__ __device__ TileCoord tile_of(int slot) const {
        if (two_group_rows == 0) return slot < all.grid_size() ? all.tile_of(slot) : TileCoord{0, 0, false};
        const int x = slot % kNumXCD, q = slot / kNumXCD;
        const int mine = first_tiles > x ? (first_tiles - x + kNumXCD - 1) / kNumXCD : 0;      // two-group tiles of this XCD
        if (q < mine) {
            const int t = q * kNumXCD + x;
            return {t / all.tiles_n, t % all.tiles_n, true};
        }
        const int s = (q - mine) * kNumXCD + x;
        if (s >= rest.grid_size()) return {0, 0, false};
        TileCoord t = rest.dealt_band_tile_of(s);
        t.m_idx += two_group_rows;
        return t;
    }
};

// Workgroups to launch for `slots` units of work (tiles, or groups x tiles) under the caller's compute-unit cap, the
// `num_sms` of the reference's persistent kernels (yan/include/gemm/fp8_gemm.cuh:40 launches num_sms blocks,
// yan/jit_kernels/utils.py:6-29 holds the cap). No cap (0, or at least `device_cus`): one workgroup per slot, and the
// hardware hands them to compute units as they free up. A cap below the device's compute units: that many workgroups,
// rounded down to a multiple of the 8 XCDs so that slot b, b + grid, b + 2 grid, ... all fall to the same XCD and the
// scheduler's per-XCD ranges keep their meaning; workgroup b then walks those slots.
__host__ __device__ inline int capped_grid(int slots, int num_sms, int device_cus) {
    if (num_sms <= 0 || num_sms >= device_cus || num_sms >= slots) return slots;
    return num_sms >= kNumXCD ? num_sms / kNumXCD * kNumXCD : num_sms;
}

// Split-K workspaces (fp8_gemm.hpp, bf16_gemm.hpp): the arrival counters take the first kSplitKCounterBytes whatever the
// problem, so that launches of different shapes and kernels can share a workspace; the largest plan of the tile heuristics
// (256 workgroups of 128 x 128 partial sums) fits kSplitKWorkspaceBytes.
constexpr size_t kSplitKCounterBytes = 16 * 1024, kSplitKWorkspaceBytes = kSplitKCounterBytes + size_t(256) * 128 * 128 * 4;

} // namespace yan
