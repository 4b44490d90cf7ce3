// Host-side check of the workgroup -> tile mapping (gemm/scheduler.hpp is __host__ __device__): built and run by
// tests/test_host_cpu.py with `hipcc --cuda-host-only`, no device involved.
//
// For a range of (tiles_m, tiles_n) it asserts that
//   * tile_of over [0, grid_size()) visits every tile exactly once and marks the remaining slots invalid
//     (reference: yan/include/gemm/scheduler.cuh:39-41, num_blocks = ceil(m/BLOCK_M) * ceil(N/BLOCK_N));
//   * under every compute-unit cap, the walk b, b + grid, b + 2 grid, ... of capped_grid() workgroups covers every slot
//     exactly once and, for grids that are multiples of 8, never leaves the XCD residue b % 8;
//   * the masked layout's slot numbering (MaskedSlots) visits every (group, tile) once, likely tile rows first, and bands
//     fitted to the height of a group lose no tile and keep a patch inside one group;
//   * the contiguous layout's slot numbering on 256-row tiles (ContiguousSlots) visits every tile once within the launched
//     slots for any number of two-group rows, and deals those rows' tiles evenly to the XCDs, first in each;
//   * the same holds in region order (operand rows long enough that the problem outgrows the memory-side cache), whose
//     choice of region is pinned for a few measured shapes.
#include "gemm/scheduler.hpp"

#include <cstdio>
#include <vector>

#define CHECK(cond)                                                                                   \
    do {                                                                                              \
        if (!(cond)) {                                                                                \
            std::printf("FAILED %s at %s:%d (m=%d n=%d bm=%d bn=%d)\n", #cond, __FILE__, __LINE__, m, n, bm, bn); \
            return 1;                                                                                 \
        }                                                                                             \
    } while (0)

int main() {
    int cases = 0, region_cases = 0;
    const int blocks[][2] = {{256, 256}, {128, 256}, {64, 16}, {256, 224}};
    for (const auto& blk : blocks) {
        const int bm = blk[0], bn = blk[1];
        for (int tm = 1; tm <= 40; tm += (tm < 12 ? 1 : 7))
            for (int tn = 1; tn <= 70; tn += (tn < 10 ? 1 : 9)) {
                // ragged sizes: the last tile of each dimension holds a single row / column
                const int m = (tm - 1) * bm + 1, n = (tn - 1) * bn + 1;
                // bytes per operand row: 0 = band order; the others put problems of 256 tiles and more whose operands
                // outgrow the 256 MB cache into region order
                for (long long row_bytes : {0ll, 4096ll, 28672ll, 262144ll}) {
                const yan::XcdTileScheduler<> sched(m, n, bm, bn, row_bytes);
                if (row_bytes == 0 || tm * tn < 256) CHECK(sched.region_rows == 0);
                if (sched.region_rows) {
                    ++region_cases;
                    CHECK(sched.region_rows * sched.region_cols == 256 && sched.region_rows % 8 == 0 && sched.region_cols % 4 == 0);
                }
                CHECK(sched.tiles_m == tm && sched.tiles_n == tn && sched.total == tm * tn);
                const int slots = sched.grid_size();
                CHECK(slots >= sched.total && slots < sched.total + yan::kNumXCD && slots % yan::kNumXCD == 0);
                std::vector<int> seen(size_t(tm) * tn, 0);
                int invalid = 0;
                for (int bid = 0; bid < slots; ++bid) {
                    const yan::TileCoord t = sched.tile_of(bid);
                    if (!t.valid) { ++invalid; continue; }
                    CHECK(t.m_idx >= 0 && t.m_idx < tm && t.n_idx >= 0 && t.n_idx < tn);
                    ++seen[size_t(t.m_idx) * tn + t.n_idx];
                }
                CHECK(invalid == slots - sched.total);
                for (int v : seen) CHECK(v == 1);
                // walks under a cap
                for (int cap : {0, 1, 3, 8, 20, 64, 100, 255, 256, 300}) {
                    const int grid = yan::capped_grid(slots, cap, 256);
                    CHECK(grid >= 1 && grid <= slots);
                    if (cap <= 0 || cap >= 256 || cap >= slots) CHECK(grid == slots);
                    else CHECK(grid <= cap && (cap < yan::kNumXCD || grid % yan::kNumXCD == 0) && grid > cap - yan::kNumXCD);
                    std::vector<int> hit(slots, 0);
                    for (int b = 0; b < grid; ++b)
                        for (int slot = b; slot < slots; slot += grid) {
                            ++hit[slot];
                            if (grid % yan::kNumXCD == 0) CHECK(slot % yan::kNumXCD == b % yan::kNumXCD);
                        }
                    for (int v : hit) CHECK(v == 1);
                }
                ++cases;
                }
            }
    }
    // bands fitted to the tile-rows of a group (grouped layouts): still every tile exactly once, and with aligned groups the
    // 32 consecutive tiles of a patch stay inside one group
    for (int rows_per_group : {1, 2, 3, 4, 5, 8, 11})
        for (int groups : {1, 4, 9})
            for (int tn : {1, 7, 16, 40}) {
                const int bm = 256, bn = 256, tm = rows_per_group * groups, m = tm * bm, n = (tn - 1) * bn + 1;
                yan::XcdTileScheduler<> sched(m, n, bm, bn);
                sched.fit_bands_to_groups(rows_per_group);
                CHECK(sched.band_height == (rows_per_group < 8 ? rows_per_group : 8));
                std::vector<int> seen(size_t(tm) * tn, 0);
                for (int bid = 0; bid < sched.grid_size(); ++bid) {
                    const yan::TileCoord t = sched.tile_of(bid);
                    if (t.valid) { CHECK(t.m_idx >= 0 && t.m_idx < tm && t.n_idx >= 0 && t.n_idx < tn); ++seen[size_t(t.m_idx) * tn + t.n_idx]; }
                }
                for (int v : seen) CHECK(v == 1);
                if (rows_per_group <= 8 && 32 % rows_per_group == 0 && tn % (32 / rows_per_group) == 0)
                    for (int t0 = 0; t0 + 32 <= sched.total; t0 += 32) {
                        const int g0 = sched.band_tile(t0).m_idx / rows_per_group;
                        for (int t = t0; t < t0 + 32; ++t) CHECK(sched.band_tile(t).m_idx / rows_per_group == g0);
                    }
                ++cases;
            }
    // the masked layout's slot numbering: every (group, tile) exactly once, the tile rows below expected_m before the others
    for (int groups : {1, 3, 8, 17})
        for (int tm = 1; tm <= 9; tm += (tm < 3 ? 1 : 3))
            for (int tn : {1, 5, 16, 33})
                for (int expected : {0, 1, 100, 257, 100000}) {
                    const int bm = 128, bn = 256, m = (tm - 1) * bm + 1, n = (tn - 1) * bn + 1;
                    const yan::MaskedSlots slots(groups, m, n, bm, bn, expected);
                    CHECK(slots.num_slots() % yan::kNumXCD == 0 && slots.num_slots() < (long long)groups * tm * tn + 2 * yan::kNumXCD);
                    std::vector<int> seen(size_t(groups) * tm * tn, 0);
                    const int likely_rows = expected <= 0 ? tm : ((expected + bm - 1) / bm < tm ? (expected + bm - 1) / bm : tm);
                    bool rest_seen = false;
                    for (int s = 0; s < slots.num_slots(); ++s) {
                        int g = -1;
                        const yan::TileCoord t = slots.tile_of(s, &g);
                        if (!t.valid) continue;
                        CHECK(g >= 0 && g < groups && t.m_idx >= 0 && t.m_idx < tm && t.n_idx >= 0 && t.n_idx < tn);
                        ++seen[(size_t(g) * tm + t.m_idx) * tn + t.n_idx];
                        if (t.m_idx >= likely_rows) rest_seen = true;
                        else CHECK(!rest_seen);
                    }
                    for (int v : seen) CHECK(v == 1);
                    ++cases;
                }
    // the contiguous layout's slot numbering on 256-row tiles (ContiguousSlots): every (row position, column) once within the
    // slots the host launches, whatever number of two-group rows the device finds; those rows' tiles come first in every
    // XCD's slots and no XCD gets two more of them than another
    for (int tm : {1, 2, 7, 8, 32, 33, 73, 128})
        for (int tn : {1, 2, 16, 28, 33})
            for (int groups : {1, 4, 16})
                for (int two : {0, 1, 2, 7, 8, 31, 64, 127}) {
                    if (two > tm) continue;
                    const int bm = 256, bn = 256, m = (tm - 1) * bm + 129, n = (tn - 1) * bn + 1;
                    const yan::ContiguousSlots slots(m, n, bm, bn, groups, two);
                    const long long num_slots = yan::ContiguousSlots::num_slots(m, n, bm, bn);
                    CHECK(num_slots % yan::kNumXCD == 0 && num_slots <= (long long)tm * tn + 2 * yan::kNumXCD);
                    std::vector<int> seen(size_t(tm) * tn, 0);
                    int first_of_xcd[yan::kNumXCD] = {0};
                    bool other_seen[yan::kNumXCD] = {false};
                    for (int s = 0; s < num_slots; ++s) {
                        const yan::TileCoord t = slots.tile_of(s);
                        if (!t.valid) continue;
                        CHECK(t.m_idx >= 0 && t.m_idx < tm && t.n_idx >= 0 && t.n_idx < tn);
                        ++seen[size_t(t.m_idx) * tn + t.n_idx];
                        if (two == 0) continue;
                        const int x = s % yan::kNumXCD;
                        if (t.m_idx < two) { CHECK(!other_seen[x]); ++first_of_xcd[x]; }
                        else other_seen[x] = true;
                    }
                    for (int v : seen) CHECK(v == 1);
                    for (int x = 0; x < yan::kNumXCD; ++x) CHECK(first_of_xcd[x] - first_of_xcd[yan::kNumXCD - 1] <= 1 && first_of_xcd[x] >= first_of_xcd[yan::kNumXCD - 1]);
                    ++cases;
                }
    // what the traffic model picks for shapes that were measured (bf16, 256 x 256 tiles)
    {
        const int m = 0, n = 0, bm = 256, bn = 256;
        const yan::XcdTileScheduler<> a(8192, 8192, 256, 256, 12288 * 2), b(8192, 4096, 256, 256, 14336 * 2),
            c(12288, 12288, 256, 256, 12288 * 2), d(8192, 8192, 256, 256, 8192 * 2), e(16384, 16384, 256, 256, 16384);
        CHECK(a.region_rows == 32 && a.rows_outer);          // the activation block stays: what band order amounts to
        CHECK(b.region_rows == 16 && c.region_rows == 32);
        CHECK(d.region_rows == 0);                           // 2 x 128 MiB of operands fit
        CHECK(e.region_rows == 32 && e.rows_outer);          // the FP8 16384^3 shape
        CHECK(region_cases > 100);
    }
    std::printf("ok %d\n", cases);
    return 0;
}
