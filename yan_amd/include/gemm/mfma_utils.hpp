// MFMA atoms for gfx950 and the wave-count helpers of the GEMM kernels.
// Takes the place of the reference's WGMMA selector (yan/include/gemm/mma_utils.cuh:17-84): there an atom is
// a 64xNx32 e4m3 warpgroup op chosen by BLOCK_N; here an atom is one wavefront-wide MFMA.
//
// Operand convention used by every kernel in this directory (64 lanes, lane l):
//   square atom of R rows:  group g = l / R,  index i = l % R
//   "row" operand   : lane holds row i,    the g-th 16-byte (bf16/f16) or 32-byte (fp8) K slice
//   "col" operand   : lane holds column i, the same K slice
//   accumulator     : lane holds column i; R == 32: rows 8*(r/4) + 4*g + r%4 for r in [0,16)
//                                          R == 16: rows 4*g + r           for r in [0,4)
// K slices are paired lane-group by lane-group, so any assignment of K bytes to (g, byte) is valid as long
// as both operands use the same one.
#pragma once

#include "utils.hpp"

namespace yan {

__device__ __forceinline__ int get_lane_id() { return threadIdx.x & (kWaveSize - 1); }

// 32x32x16, bf16 in, fp32 accumulate: 8 passes, 16 accumulator registers per lane.
struct MfmaBF16_32x32x16 {
    static constexpr int R = 32, K_BYTES = 32, ACC = 16;
    using Frag = bf16x8;
    using Acc  = f32x16;
    __device__ __forceinline__ static Acc mma(Frag rows, Frag cols, Acc c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(rows, cols, c, 0, 0, 0);
    }
};

// Same shape for IEEE half inputs.
struct MfmaF16_32x32x16 {
    static constexpr int R = 32, K_BYTES = 32, ACC = 16;
    using Frag = f16x8;
    using Acc  = f32x16;
    __device__ __forceinline__ static Acc mma(Frag rows, Frag cols, Acc c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(rows, cols, c, 0, 0, 0);
    }
};

// 16x16x32, bf16 / f16 in, fp32 accumulate: 4 passes, 4 accumulator registers per lane; a lane holds 8 consecutive
// K values (16 bytes) of row l % 16, K group l / 16.
struct MfmaBF16_16x16x32 {
    static constexpr int R = 16, K_BYTES = 64, ACC = 4;
    using Frag = bf16x8;
    using Acc  = f32x4;
    __device__ __forceinline__ static Acc mma(Frag rows, Frag cols, Acc c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(rows, cols, c, 0, 0, 0);
    }
};

struct MfmaF16_16x16x32 {
    static constexpr int R = 16, K_BYTES = 64, ACC = 4;
    using Frag = f16x8;
    using Acc  = f32x4;
    __device__ __forceinline__ static Acc mma(Frag rows, Frag cols, Acc c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(rows, cols, c, 0, 0, 0);
    }
};

// 16x16x128 over OCP e4m3 bytes (cbsz = blgp = 0 selects e4m3 for both operands; zero scale operands select
// the unscaled instruction): 8 passes, a whole 128-deep scale block per instruction, 4 accumulator registers.
struct MfmaFP8_16x16x128 {
    static constexpr int R = 16, K_BYTES = 128, ACC = 4;
    using Frag = i32x8;
    using Acc  = f32x4;
    __device__ __forceinline__ static Acc mma(Frag rows, Frag cols, Acc c) {
        return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(rows, cols, c, 0, 0, 0, 0, 0, 0);
    }
};

// 32x32x64 over OCP e4m3 bytes: 16 passes, half a scale block per instruction.
struct MfmaFP8_32x32x64 {
    static constexpr int R = 32, K_BYTES = 64, ACC = 16;
    using Frag = i32x8;
    using Acc  = f32x16;
    __device__ __forceinline__ static Acc mma(Frag rows, Frag cols, Acc c) {
        return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(rows, cols, c, 0, 0, 0, 0, 0, 0);
    }
};

// Waves per workgroup for a macro tile: two waves per SIMD (8 in all) from 256 x 128 up, and from 64 x 64 up when
// both sides are whole copy passes of eight waves (64 rows); one wave per SIMD otherwise. A wave gets one
// global-to-LDS copy instruction through per ~50 ns whatever its width, so four waves pull at most ~59 GB/s per CU
// in the row-strided pattern of the operand copies and eight ~103 GB/s: measured, the 128 x 128 tile runs 12-20 %
// faster with eight waves than with four, 64 x 128 and 64 x 64 4-7 %.
__host__ __device__ constexpr int get_num_waves(int block_m, int block_n) {
    if (block_m * block_n >= 256 * 128) return 8;
    return (block_m * block_n >= 64 * 64 && block_m % 64 == 0 && block_n % 64 == 0) ? 8 : 4;
}

// How many of a workgroup's `num_waves` waves sit side by side along n (the rest stack along m): the split whose
// per-wave slab is a whole number of `atom`-row atoms, holds at most `max_slab` outputs and reads the fewest LDS
// rows per k-tile (slab_n + slab_m); ties go to the wider slab along n. Returns 0 when nothing fits.
__host__ __device__ constexpr int pick_waves_n(int block_m, int block_n, int num_waves, int atom, int max_slab) {
    int best = 0, best_cost = 1 << 30;
    for (int wn = 1; wn <= num_waves; wn *= 2) {
        const int wm = num_waves / wn;
        if (block_n % (wn * atom) != 0 || block_m % (wm * atom) != 0) continue;
        const int slab_n = block_n / wn, slab_m = block_m / wm;
        if (slab_n * slab_m > max_slab) continue;
        if (slab_n + slab_m < best_cost) { best = wn; best_cost = slab_n + slab_m; }
    }
    return best;
}

} // namespace yan
