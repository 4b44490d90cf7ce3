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
// Workgroup `bid` therefore runs on XCD `bid % 8`. Every XCD gets one contiguous range of the tile
// sequence, and the sequence itself walks bands of GROUP_M tile-rows column by column, so the 32 tiles an
// XCD has in flight form a compact GROUP_M x 4 patch whose A and B panels are shared through that L2.
template <int GROUP_M = 8>
struct XcdTileScheduler {
    int tiles_m, tiles_n, total, per_xcd;

    __host__ __device__ XcdTileScheduler(int m, int n, int block_m, int block_n) {
        tiles_m = ceil_div(m, block_m);
        tiles_n = ceil_div(n, block_n);
        total   = tiles_m * tiles_n;
        per_xcd = ceil_div(total, kNumXCD);
    }

    __host__ __device__ int grid_size() const { return per_xcd * kNumXCD; }

    __host__ __device__ TileCoord tile_of(int bid) const {
        const int t = (bid % kNumXCD) * per_xcd + bid / kNumXCD;
        if (t >= total) return {0, 0, false};
        const int band      = GROUP_M * tiles_n;
        const int first_m   = (t / band) * GROUP_M;
        const int band_rows = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
        const int in_band   = t % band;
        return {first_m + in_band % band_rows, in_band / band_rows, true};
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

} // namespace yan
