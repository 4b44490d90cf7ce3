// out[m,n] = sum_kb sA[m,kb] * sB[n/128,kb] * sum_{t<128} A8[m,128kb+t] * B8[n,128kb+t]   (e4m3 x e4m3 -> fp32 -> bf16)
//
// The block-scaled FP8 GEMM of the reference's yan/include/gemm/fp8_gemm.cuh (template parameters :32-39,
// kernel signature :40-46, BLOCK_K == 128 :48, one A scale per row and K block and one or two B scales per tile
// and K block :55-61), which in the reference is an unfinished Hopper kernel built on TMA descriptors, cluster
// barriers and warpgroup MMAs. This is a different kernel for gfx950:
//   * macro tile BLOCK_M x BLOCK_N x 128 (one scale block per k-tile, 128-byte rows); 8 waves, two per SIMD, for
//     the tiles from 256 x 128 up and for the tiles from 64 x 64 up whose sides are multiples of 64 (get_num_waves in
//     mfma_utils.hpp), so one wave's scale arithmetic and LDS traffic hide under the other's MFMAs and eight waves issue
//     the copies; 4 waves otherwise;
//   * HBM -> LDS with buffer_load ... lds (tile_io.hpp) into two LDS stages for the 256-row tiles (160 to 256 columns) and
//     into a ring of 3 to 12 stages for the smaller tiles, which run problems bound by operand streaming; the tiles of the
//     decode shapes (32 x 32, 64 x 32) consume their ring four k-tiles per barrier, with four more waves that only copy;
//   * 16x16x128 e4m3 MFMAs: one instruction covers a whole scale block, starts from a zero accumulator and
//     yields 4 partial sums per lane, which the VALU folds into the running fp32 sums as acc += partial * s,
//     s = sA * sB. Weights feed the MFMA row operand and activations the column operand, so a lane only ever
//     meets one activation row per atom: one sA per lane per atom per K block, and sB is wave-uniform;
//   * the running sums stay in architectural VGPRs (the VALU cannot address AGPRs): 128 per wave;
//   * the output leaves through LDS: each wave turns its slab round through the stage that was consumed last and stores
//     16 bytes per lane in row runs of 2 * WTN bytes (non-temporal when the output is larger than the L2s together,
//     except in the persistent walk, whose stores are plain);
//   * the plain GEMM on the 256-row tiles is a persistent walk: one workgroup per compute unit takes tile after tile and
//     overlaps the seams (fp8_gemm_walk); every other case runs a workgroup per tile, or a plain loop under a cap;
//   * problems with long K and fewer tiles than compute units split K over SPLIT_K workgroups per tile on the ring tiles
//     (fp8_gemm_split_k_kernel, the `split` of the reference's tile/split heuristics): the parts meet in a caller-provided
//     workspace, the last to arrive adds them up in the order of their K ranges and stores the tile (fp8_meet_partials);
//   * m is a run-time argument with tails predicated; N and K are compile-time in the JIT kernels and run-time (template
//     arguments 0) in the ahead-of-time library;
//   * grouped (mixture-of-experts) layouts, the reference's GemmType::GroupedContiguous / GroupedMasked hooks
//     (yan/include/gemm/scheduler.cuh:7-11,31-48, `int* grouped_layout` of fp8_gemm.cuh:41): every output tile
//     belongs to one group, which picks the [N, K] weight matrix and its scale table; the rest of the kernel
//     does not know about groups.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp8.h>

#include "utils.hpp"
#include "mfma_utils.hpp"
#include "scheduler.hpp"
#include "tile_io.hpp"

namespace yan {

// K-tiles a tile's ring is consumed by per barrier (1: one at a time) and the waves its workgroup is launched with.
// Tiles of one or two atoms per wave (the decode shapes) with a ring of 12 stages take four k-tiles per barrier, and
// four more waves that only copy: a wave gets one copy instruction through per ~50 ns, and three per k-tile on each
// of four waves (activations, weights, scales) was what bounded these tiles.
__host__ __device__ constexpr int fp8_ring_group(int block_m, int block_n, int stages) {
    return ((block_m == 32 || block_m == 64) && block_n == 32 && stages >= 12 && stages % 4 == 0) ? 4 : 1;
}
__host__ __device__ constexpr int fp8_launch_waves(int block_m, int block_n, int stages) {
    return fp8_ring_group(block_m, block_n, stages) > 1 ? 8 : get_num_waves(block_m, block_n);
}

template <int BLOCK_M, int BLOCK_N>
struct Fp8TileConfig {
    static constexpr int NUM_WAVES = get_num_waves(BLOCK_M, BLOCK_N);
    static constexpr int WAVES_N   = pick_waves_n(BLOCK_M, BLOCK_N, NUM_WAVES, 16, 128 * 64);
    static_assert(WAVES_N > 0, "no wave layout fits this tile");
    static constexpr int WAVES_M   = NUM_WAVES / WAVES_N;
    static constexpr int WTN = BLOCK_N / WAVES_N, WTM = BLOCK_M / WAVES_M;
    static_assert(WTN % 16 == 0 && WTM % 16 == 0, "wave slab must be a whole number of 16x16 atoms");
    static_assert(WTN * WTM <= 128 * 64, "running sums must fit 128 VGPRs per lane");
    // A slab that divides a 128-wide scale block never straddles two of them.
    static constexpr bool UNIFORM_SCALE_B = (128 % WTN == 0);
    // Number of 128-wide scale blocks a slab of 16-aligned start can touch.
    static constexpr int  SCALE_B_PER_SLAB = UNIFORM_SCALE_B ? 1 : (WTN + 112) / 128 + 1;
    // LDS rows of the two operand tiles: whole copy passes (tile_io.hpp), i.e. rounded up to 8 rows per wave.
    static constexpr int  LDS_ROWS_A = TileStager<BLOCK_M, NUM_WAVES>::PADDED_ROWS, LDS_ROWS_B = TileStager<BLOCK_N, NUM_WAVES>::PADDED_ROWS;
    static constexpr int  LDS_BYTES = 2 * (LDS_ROWS_A + LDS_ROWS_B) * kRowBytes;
    static_assert(LDS_BYTES <= 160 * 1024, "two stages must fit the 160 KB LDS");
    // Ring of more than two stages (tiles below 256 x 256, where one k-tile in flight does not cover the memory
    // latency of an operand-streaming problem): a stage also carries the k-tile's activation scales (one copy
    // instruction moves 64 of them; a 32-row tile uses the first 32).
    static constexpr int  RING_SCALE_BYTES = ceil_div(BLOCK_M * 4, 1024) * 1024;
    static constexpr int  RING_STAGE_BYTES = (LDS_ROWS_A + LDS_ROWS_B) * kRowBytes + RING_SCALE_BYTES;
    static constexpr bool RING_CAPABLE = BLOCK_M % 32 == 0 && (BLOCK_M / 8) % NUM_WAVES == 0 && BLOCK_N % 16 == 0;
    // At most 8 stages, 12 for the narrow tiles of the decode shapes (16 or 32 weight rows per workgroup): those have next
    // to nothing to compute per k-tile and run at the rate their compute unit takes bytes in, which needs many k-tiles in
    // flight (a stage is only 9 to 13 KB there). Measured with every unit pulling: about 60 GB/s per unit whatever the
    // tile, so the tile to prefer is the one that moves the fewest bytes per output, 32 x 32 for a 64-row problem.
    static constexpr int  RING_DEPTH_CAP = BLOCK_N <= 32 ? 12 : 8;
    static constexpr int  MAX_RING_STAGES = RING_CAPABLE ? (160 * 1024 / RING_STAGE_BYTES < RING_DEPTH_CAP ? 160 * 1024 / RING_STAGE_BYTES : RING_DEPTH_CAP) : 2;
};

// The two LDS stages of the 256-row tiles (operand tiles of Fp8TileConfig::LDS_ROWS_A / LDS_ROWS_B rows each), declared
// once in the kernel and handed to whichever of its bodies runs; unused by the ring tiles, which declare their own ring.
struct Fp8TwoStages {
    uint8_t *a0, *b0, *a1, *b1;
};

// The MFMA operand of a 16-row atom whose rows start at `atom_rows` in a staged tile: lane group g holds bytes
// [32 g, 32 g + 32) of its row, two 16-byte chunks at the offsets frag_offset<16> gives for chunks 2g and 2g + 1.
__device__ __forceinline__ i32x8 fp8_read_frag(const uint8_t* atom_rows, int off0, int off1) {
    const i32x4 lo = *reinterpret_cast<const i32x4*>(atom_rows + off0);
    const i32x4 hi = *reinterpret_cast<const i32x4*>(atom_rows + off1);
    return i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

// One k-tile of a wave's slab: TN x TM atoms, software-pipelined by hand. `pa` / `pb` are the slab's first activation
// and weight rows in the staged tile. Step t issues the MFMA of atom t (fresh zero accumulator) and folds in the partial
// sums of atom t - DEPTH, whose MFMA has retired by then; the fragment of weight rows i+1 is fetched while rows i are
// being multiplied; `row_hook(i)` runs once per row of atoms and is where the copies of the next k-tile are started.
// sched_barrier keeps the compiler from regrouping the steps (it would otherwise hoist every MFMA and need a register
// per partial sum). `sa`: the activation scales of this lane's row in each of the TM atoms; `sb`: the weight scales of
// the one or two 128-wide blocks the slab touches, `rows_in_first_block` rows of atoms lying in the first.
template <typename Cfg, int TN, int TM, int NB, typename RowHook>
__device__ __forceinline__ void
fp8_compute_k_tile(f32x4 (&acc)[TN][TM], const uint8_t* pa, const uint8_t* pb, const float (&sa)[TM], const float (&sb)[NB],
                   int rows_in_first_block, int off0, int off1, RowHook&& row_hook) {
    using Atom = MfmaFP8_16x16x128;
    // A fold three steps behind its MFMA: at two the fold still waits for the MFMA now and then (a build whose folds do not
    // depend on the MFMAs at all runs 3-4 % faster), at three 1-1.7 % of that is back on the 256-row tiles and 4 % on
    // 64 x 128 (cfg3 174.4 -> 172.5 us, 8192 x 7168 x 7168 333.0 -> 327.5, 512 x 4096 x 2048 9.83 -> 9.40); four and five
    // steps, with a ring of eight partial sums, are no better than three.
    constexpr int T = TN * TM, DEPTH = 3, RING = 4;
    static_assert(DEPTH < RING);
    i32x8 mf[TM], nf[2];
    nf[0] = fp8_read_frag(pb, off0, off1);
#pragma unroll
    for (int j = 0; j < TM; ++j) mf[j] = fp8_read_frag(pa + j * 16 * kRowBytes, off0, off1);
    float s[TM];
    [[maybe_unused]] float s_first[TM], s_second[TM];
    f32x4 p[RING];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < T + DEPTH; ++t) {
        if (t < T) {
            const int i = t / TM, j = t % TM;
            if (j == 1 % TM) row_hook(i);
            if (j == 0 && i + 1 < TN) nf[(i + 1) & 1] = fp8_read_frag(pb + (i + 1) * 16 * kRowBytes, off0, off1);
            p[t % RING] = Atom::mma(nf[i & 1], mf[j], f32x4{0.f, 0.f, 0.f, 0.f});
        }
        if (t >= DEPTH) {
            const int u = t - DEPTH, i = u / TM, j = u % TM;
            if constexpr (Cfg::UNIFORM_SCALE_B) {
                if (u == 0) {
#pragma unroll
                    for (int jj = 0; jj < TM; ++jj) s[jj] = sa[jj] * sb[0];
                }
            } else if (j == 0) {
                // A slab that is not a divisor of 128 wide crosses at most one boundary between weight-scale
                // blocks: rows of atoms below `rows_in_first_block` take block 0's scale, the others block 1's.
                // Both products are formed once per k-tile and each row picks its own with a bit select under a
                // wave-uniform mask: no branch, so the steps stay in one basic block.
                static_assert(NB == 2, "a slab narrower than 128 touches at most two scale blocks");
                if (i == 0) {
#pragma unroll
                    for (int jj = 0; jj < TM; ++jj) { s_first[jj] = sa[jj] * sb[0]; s_second[jj] = sa[jj] * sb[1]; }
                }
                const uint32_t pick_second = i >= rows_in_first_block ? 0xffffffffu : 0u;
#pragma unroll
                for (int jj = 0; jj < TM; ++jj)
                    s[jj] = __builtin_bit_cast(float, (__builtin_bit_cast(uint32_t, s_second[jj]) & pick_second) |
                                                      (__builtin_bit_cast(uint32_t, s_first[jj]) & ~pick_second));
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = __builtin_fmaf(p[u % RING][r], s[j], acc[i][j][r]);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

// A wave's slab of sums out to memory as bf16. The 4 registers of atom (i, j) are n = n_slab + 16i + 4g + {0..3} of row
// m = m_slab + 16j + col; stored straight from there a wave instruction writes 16 rows x 32 bytes. With `region` (LDS
// of 16 * (2 WTN + 16) bytes that nobody else touches) the slab instead turns round through it, 16 rows at a time, and
// is stored 16 bytes per lane in runs of 2 * WTN consecutive bytes per row; rows are 2 * WTN + 16 bytes apart in LDS,
// which spreads the 8-byte writes of 16 rows over the banks. STAGED = false: the direct stores, `region` unused.
// Rows outside [row_lo, row_hi) and columns from n on are not stored. `rsrc_out` addresses the output tile that starts
// at (m0, n0); `lane` should be an opaque copy of the lane number made after the main loop, which has no registers to
// spare for addresses computed ahead of time.
template <typename Cfg, bool STAGED, int TN, int TM>
__device__ __forceinline__ void
fp8_store_slab(const f32x4 (&acc)[TN][TM], uint8_t* region, __amdgpu_buffer_rsrc_t rsrc_out, int m_slab, int n_slab, int m0, int n0,
               int row_lo, int row_hi, int n, bool stream_out, int lane) {
    const int col = lane % 16, g = lane / 16;
    if constexpr (STAGED) {
        {
            static_assert(Cfg::WTN >= 32);
            constexpr int PITCH = Cfg::WTN * 2 + 16;
            constexpr int LANES_PER_ROW = Cfg::WTN / 8, ROWS_PER_STORE = kWaveSize / LANES_PER_ROW, STORES = ceil_div(16, ROWS_PER_STORE);
            const int r_in = lane / LANES_PER_ROW, c = lane % LANES_PER_ROW;
            const int nn = n_slab + 8 * c;
#pragma unroll
            for (int j = 0; j < TM; ++j) {
#pragma unroll
                for (int i = 0; i < TN; ++i)
                    *reinterpret_cast<bf16x4*>(region + col * PITCH + (16 * i + 4 * g) * 2) = pack4(acc[i][j], __bf16{});
#pragma unroll
                for (int q = 0; q < STORES; ++q) {
                    const int row = ROWS_PER_STORE * q + r_in, mm = m_slab + 16 * j + row;
                    const i32x4 v = *reinterpret_cast<const i32x4*>(region + row * PITCH + c * 16);
                    // a slab width that does not divide 64 lanes leaves the last lanes, and rows past 16, without work
                    const bool live = mm >= row_lo && mm < row_hi && nn < n && r_in < ROWS_PER_STORE && row < 16;
                    if (live) buffer_store_16(v, rsrc_out, uint32_t((mm - m0) * n + nn - n0) * 2u, stream_out);
                }
                __builtin_amdgcn_sched_barrier(0);      // one 16-row pass at a time: the registers are full of sums
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            const int mm = m_slab + j * 16 + col;
            if (mm < row_lo || mm >= row_hi) continue;
#pragma unroll
            for (int i = 0; i < TN; ++i) {
                const int nn = n_slab + i * 16 + 4 * g;
                if (nn < n) buffer_store_8(pack4(acc[i][j], __bf16{}), rsrc_out, uint32_t((mm - m0) * n + nn - n0) * 2u, stream_out);
            }
        }
    }
}

// Normal:            lhs [m, K], rhs [N, K], out [m, N]; grouped_layout unused.
// GroupedContiguous: lhs [m, K] is the concatenation of the groups' rows, every group padded to a multiple of 128
//                    rows (BLOCK_M divides 128); grouped_layout[i] is the group of row i, negative for padding rows,
//                    whose tiles are skipped; rhs [G, N, K], rhs_scales [G, ceil(N/128), K/128].
// GroupedMasked:     lhs [G, m, K], out [G, m, N], rhs as above; only the first grouped_layout[g] rows of group g
//                    are computed; lhs_scales of group g start at g * sa_stride_g floats. Slots are numbered by
//                    MaskedSlots: the tile rows below `expected_m` of all groups first.
// Where the SPLIT_K parts of a tile meet (meet_partials in tile_io.hpp): the wave's TN x TM atoms of four sums each.
template <int SPLIT_K, int NW, int TN, int TM>
__device__ __forceinline__ bool
fp8_meet_partials(f32x4 (&acc)[TN][TM], float* __restrict__ partials, unsigned* __restrict__ counters, int tile_slot, int split, int wave, int lane) {
    return meet_partials<SPLIT_K, NW, TN * TM>([&](int v) -> f32x4& { return acc[v / TM][v % TM]; }, partials, counters, tile_slot, split, wave, lane);
}

// Contiguous groups on 256-row tiles: which tile rows hold two groups (they go first in the launch order, ContiguousSlots in
// scheduler.hpp) is in `grouped_layout`, on the device; every wave works it out for itself, 64 tile rows at a time with a
// row per lane. Bit `lane` of the result: tile row 64 * chunk + lane has a group in either half, and not the same.
__device__ __forceinline__ unsigned long long
two_group_rows_of_chunk(const int* __restrict__ grouped_layout, int m, int tiles_m, int chunk, int lane) {
    const int row = chunk * kWaveSize + lane, m0 = row * 256;
    bool yes = false;
    if (row < tiles_m && m0 + 128 < m) {
        const int g0 = grouped_layout[m0], g1 = grouped_layout[m0 + 128];
        yes = g0 >= 0 && g1 >= 0 && g0 != g1;
    }
    return __ballot(yes);
}

__device__ __forceinline__ int
count_two_group_rows(const int* __restrict__ grouped_layout, int m, int tiles_m, int lane) {
    int count = 0;
    for (int c = 0; c < ceil_div(tiles_m, kWaveSize); ++c) count += __popcll(two_group_rows_of_chunk(grouped_layout, m, tiles_m, c, lane));
    return count;
}

// The tile row at position `pos` of the order "two-group rows first, then the others, either kind ascending". Wave-uniform.
__device__ __forceinline__ int
contiguous_row_at(const int* __restrict__ grouped_layout, int m, int tiles_m, int count, int pos, int lane) {
    const bool among_two = pos < count;
    int rank = among_two ? pos : pos - count;
    for (int c = 0; c < ceil_div(tiles_m, kWaveSize); ++c) {
        const int rows_here = min(kWaveSize, tiles_m - c * kWaveSize);
        const unsigned long long all = rows_here == 64 ? ~0ull : ((1ull << rows_here) - 1);
        const unsigned long long two = two_group_rows_of_chunk(grouped_layout, m, tiles_m, c, lane), mask = among_two ? two : (~two & all);
        const int here = __popcll(mask);
        if (rank < here) {
            const bool mine = ((mask >> lane) & 1) && __popcll(mask & ((1ull << lane) - 1)) == rank;
            const unsigned long long found = __ballot(mine);
            return found ? c * kWaveSize + __ffsll((long long)found) - 1 : pos;
        }
        rank -= here;
    }
    return pos;         // not reached: pos < tiles_m
}

// STAGES: 2 = two LDS stages with the next k-tile's scales in registers; 3.. = a ring of that many stages.
// One output tile (one slot of the launch: `bid` is what blockIdx.x would be with a workgroup per slot).
// EXTERNAL_RING: the ring of a tile with STAGES > 2 lives in `ring_lds` (LDS the caller declared, 1024-byte aligned, at least
// STAGES * Fp8TileConfig::RING_STAGE_BYTES) instead of an array of this function's own: for kernels that hold two kinds of
// tile and run one of them (fp8_gemm_contiguous_rows_kernel).
// EXPLICIT_TILE: `bid` names the tile itself, row-major over the tile grid (m_idx * tiles_n + n_idx), for callers that order the
// tiles themselves.
template <int SHAPE_N, int SHAPE_K, int BLOCK_M, int BLOCK_N, GemmType kGemmType, int STAGES, int SPLIT_K = 1, bool EXTERNAL_RING = false,
          bool EXPLICIT_TILE = false>
__device__ __forceinline__ void
fp8_gemm_tile(const uint8_t* __restrict__ lhs, const float* __restrict__ lhs_scales,
              const uint8_t* __restrict__ rhs, const float* __restrict__ rhs_scales,
              __bf16* __restrict__ out, int m, int n_rt, int k_rt, int sa_stride_m, int sa_stride_k,
              const int* __restrict__ grouped_layout, int sa_stride_g, int bid, int num_groups, int expected_m, Fp8TwoStages two_stages,
              float* __restrict__ partials = nullptr, unsigned* __restrict__ counters = nullptr, uint8_t* ring_lds = nullptr) {
    using Cfg  = Fp8TileConfig<BLOCK_M, BLOCK_N>;
    using Atom = MfmaFP8_16x16x128;
    // NW waves compute (and copy); LW are launched: the extra ones of the decode tiles only copy.
    constexpr int NW = Cfg::NUM_WAVES, LW = fp8_launch_waves(BLOCK_M, BLOCK_N, STAGES), TN = Cfg::WTN / 16, TM = Cfg::WTM / 16;
    constexpr int NB = Cfg::SCALE_B_PER_SLAB;
    static_assert(SHAPE_K % 128 == 0 && SHAPE_N % 4 == 0);
    // SHAPE_N / SHAPE_K == 0 selects the run-time sizes (ahead-of-time library); the JIT bakes them in.
    const int N = SHAPE_N ? SHAPE_N : n_rt, K = SHAPE_K ? SHAPE_K : k_rt;
    const int NUM_K_BLOCKS = K / 128, NUM_N_BLOCKS = ceil_div(N, 128);

    static_assert(STAGES == 2 || (STAGES >= 3 && STAGES <= Cfg::MAX_RING_STAGES), "no ring of this depth for this tile");

    // SPLIT_K > 1: launch slot `bid` is part `bid % SPLIT_K` of tile slot `bid / SPLIT_K`: the k-tiles [kb_lo, kb_hi) of it.
    int kb_lo = 0, kb_hi = NUM_K_BLOCKS;
    [[maybe_unused]] int split = 0;
    if constexpr (SPLIT_K > 1) {
        static_assert(kGemmType == GemmType::Normal && STAGES > 2, "K is split for plain GEMMs on ring tiles");
        split = bid % SPLIT_K;
        bid /= SPLIT_K;
        const int per = ceil_div(NUM_K_BLOCKS, SPLIT_K);
        kb_lo = min(split * per, NUM_K_BLOCKS);
        kb_hi = min(kb_lo + per, NUM_K_BLOCKS);
    }
    [[maybe_unused]] const int tile_slot = bid;

    // a plain GEMM whose operands outgrow the memory-side cache walks its tiles in region order (scheduler.hpp)
    XcdTileScheduler<> sched(m, N, BLOCK_M, BLOCK_N, kGemmType == GemmType::Normal ? (long long)K : 0);
    // contiguous groups of equal size start on band boundaries when the bands are as tall as a group (or divide one)
    if constexpr (kGemmType == GemmType::GroupedContiguous) sched.fit_bands_to_groups(sched.tiles_m / max(num_groups, 1));
    TileCoord tile;
    if constexpr (EXPLICIT_TILE) {
        static_assert(kGemmType != GemmType::GroupedMasked);
        tile = TileCoord{bid / sched.tiles_n, bid % sched.tiles_n, bid >= 0 && bid < sched.total};
    } else if constexpr (kGemmType == GemmType::GroupedMasked) {
        int group;
        tile = MaskedSlots(num_groups, m, N, BLOCK_M, BLOCK_N, expected_m).tile_of(bid, &group);
        lhs        += size_t(group) * m * K;
        lhs_scales += size_t(group) * sa_stride_g;
        out        += size_t(group) * m * N;
        rhs        += size_t(group) * N * K;
        rhs_scales += size_t(group) * NUM_N_BLOCKS * NUM_K_BLOCKS;
        m = min(m, grouped_layout[group]);        // rows of this group that exist; tiles past them leave at once
    } else if constexpr (kGemmType == GemmType::GroupedContiguous && BLOCK_M == 256) {
        const int two_group_rows = count_two_group_rows(grouped_layout, m, sched.tiles_m, get_lane_id());
        tile = ContiguousSlots(m, N, BLOCK_M, BLOCK_N, num_groups, two_group_rows).tile_of(bid);
        if (tile.valid && two_group_rows) tile.m_idx = contiguous_row_at(grouped_layout, m, sched.tiles_m, two_group_rows, tile.m_idx, get_lane_id());
    } else {
        tile = sched.tile_of(bid);
    }
    if (!tile.valid) return;
    const int m0 = tile.m_idx * BLOCK_M, n0 = tile.n_idx * BLOCK_N;
    if (m0 >= m) return;
    // Contiguous groups are padded to 128 rows. A tile of up to 128 rows lies in one group. A 256-row tile may
    // hold two: it then makes two passes over K, one per 128-row half, each with its own group's weights and
    // storing only its half (rare when groups are long, and long groups are when 256-row tiles pay off).
    constexpr bool kTwoHalves = kGemmType == GemmType::GroupedContiguous && BLOCK_M == 256;
    int num_passes = 1, pass_group[2] = {0, 0}, pass_lo[2] = {m0, m0}, pass_hi[2] = {m, m};
    if constexpr (kGemmType == GemmType::GroupedContiguous) {
        static_assert(128 % BLOCK_M == 0 || BLOCK_M == 256, "tiles are 128-row blocks, parts of one, or two of them");
        const int g0 = grouped_layout[m0];
        const int g1 = (kTwoHalves && m0 + 128 < m) ? grouped_layout[m0 + 128] : g0;
        if (g0 == g1) {
            if (g0 < 0) return;
            pass_group[0] = g0;
        } else {
            // constant indices only: an index computed at run time would put these arrays into scratch memory
            const bool first = g0 >= 0, second = g1 >= 0;
            if (!first && !second) return;
            if (first) { pass_group[0] = g0; pass_hi[0] = m0 + 128; }
            if (second && first)  { pass_group[1] = g1; pass_lo[1] = m0 + 128; }
            if (second && !first) { pass_group[0] = g1; pass_lo[0] = m0 + 128; }
            num_passes = int(first) + int(second);
        }
    }
    const uint8_t* const rhs_all = rhs;
    const float* const rhs_scales_all = rhs_scales;

    const int lane = get_lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const int wn = wave % Cfg::WAVES_N, wm = wave / Cfg::WAVES_N;
    const int g = lane / 16, col = lane % 16;
    const int m_slab = m0 + wm * Cfg::WTM, n_slab = n0 + wn * Cfg::WTN;

    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(lhs, uint32_t(m) * K);
    __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(rhs, uint32_t(N) * K);
    // copies of k-tiles past the end of the range keep the count of instructions in flight and move nothing
    const __amdgpu_buffer_rsrc_t rsrc_none = make_rsrc(lhs, 0);
    TileStager<BLOCK_M, NW> stage_a;
    TileStager<BLOCK_N, NW> stage_b;
    stage_a.init(m0, K, wave, lane);
    stage_b.init(n0, K, wave, lane);

    // Activation scales through a descriptor as well: element (row, kb) at (row*stride_m + kb*stride_k) floats.
    // Atom j of the slab covers rows m_slab + 16j + col; rows past m read as 0 or as some other row's scale,
    // either of which only ever multiplies the zero partial sums of a row that is never stored.
    const uint32_t sa_bytes = (uint32_t(m - 1) * sa_stride_m + uint32_t(NUM_K_BLOCKS - 1) * sa_stride_k + 1) * 4;
    const __amdgpu_buffer_rsrc_t rsrc_sa = make_rsrc(lhs_scales, sa_bytes);
    const uint32_t sa_voff = uint32_t(m_slab + col) * sa_stride_m * 4;
    // Weight scales: rows base_blk .. base_blk+NB-1 of the [N/128, K/128] table cover the slab.
    const int base_blk = n_slab / 128;
    [[maybe_unused]] const int rows_in_first_block = (128 - (n_slab & 127)) / 16;     // only for slabs that straddle blocks

    const int off0 = frag_offset<16>(lane, 2 * g), off1 = frag_offset<16>(lane, 2 * g + 1);
    auto read_frag = [&](const uint8_t* atom_rows) { return fp8_read_frag(atom_rows, off0, off1); };

    f32x4 acc[TN][TM];

    float sa_next[TM];     // activation scales of the k-tile in flight
    float sb_next[NB];     // weight scales of the k-tile in flight (wave-uniform)
    auto load_weight_scales = [&](int kb) {
#pragma unroll
        for (int b = 0; b < NB; ++b) sb_next[b] = rhs_scales[min(base_blk + b, NUM_N_BLOCKS - 1) * NUM_K_BLOCKS + kb];
    };
    auto load_scales = [&](int kb) {
#pragma unroll
        for (int j = 0; j < TM; ++j)
            sa_next[j] = buffer_load_f32(rsrc_sa, sa_voff, (kb * sa_stride_k + j * 16 * sa_stride_m) * 4);
        load_weight_scales(kb);
    };

    // One k-tile staged at (la, lb): fp8_compute_k_tile on this wave's slab.
    auto compute_tile = [&](const uint8_t* la, const uint8_t* lb, const float (&sa)[TM], const float (&sb)[NB],
                            auto&& row_hook) {
        fp8_compute_k_tile<Cfg>(acc, la + wm * Cfg::WTM * kRowBytes, lb + wn * Cfg::WTN * kRowBytes, sa, sb, rows_in_first_block,
                                off0, off1, row_hook);
    };

    // Two LDS stages, one k-tile (= one scale block) of prefetch; the scales of the next block travel in
    // registers alongside. The copies of the next k-tile are not issued in one burst after the barrier (the
    // memory pipeline takes ~16 cycles per instruction and both waves of every SIMD would sit in its queue while
    // the matrix core idles): they are handed out a few at a time over the first half of the rows of atoms, which
    // still leaves them more than half a k-tile of MFMA time to land. The steady-state body is branch-free (a copy
    // past the last k-tile reads bytes that are never consumed, or zeros past the end of the matrix), which keeps
    // each MFMA/FMA step where it was written.
    using StA = TileStager<BLOCK_M, NW>;
    using StB = TileStager<BLOCK_N, NW>;
    constexpr int NUM_COPIES = StA::PASSES + StB::PASSES, SPREAD_ROWS = TN >= 2 ? TN / 2 : 1;
    float sa_cur[TM], sb_cur[NB];
    // A pass over one 128-row half of a 256-row tile does not fetch the other half of the activation tile: the copy passes of
    // those rows (the first or the second half of them) go through the empty descriptor and move zeros.
    [[maybe_unused]] __amdgpu_buffer_rsrc_t rsrc_a_half[2] = {rsrc_a, rsrc_a};
    static_assert(!kTwoHalves || StA::PASSES % 2 == 0);
    auto k_step = [&](int kb, const uint8_t* a_cur, const uint8_t* b_cur, uint8_t* a_nxt, uint8_t* b_nxt) {
#pragma unroll
        for (int j = 0; j < TM; ++j) sa_cur[j] = sa_next[j];
#pragma unroll
        for (int b = 0; b < NB; ++b) sb_cur[b] = sb_next[b];
        wait_for_copies();
        __syncthreads();
        load_scales(min(kb + 1, NUM_K_BLOCKS - 1));
        compute_tile(a_cur, b_cur, sa_cur, sb_cur, [&](int row) {
#pragma unroll
            for (int d = 0; d < NUM_COPIES; ++d) {
                if (d * SPREAD_ROWS / NUM_COPIES != row) continue;
                if (d < StA::PASSES) stage_a.issue_pass(kTwoHalves ? rsrc_a_half[d * 2 / StA::PASSES] : rsrc_a, a_nxt, (kb + 1) * kRowBytes, wave, d);
                else stage_b.issue_pass(rsrc_b, b_nxt, (kb + 1) * kRowBytes, wave, d - StA::PASSES);
            }
        });
    };
    // The staged epilogue (below) turns the slab round through the LDS stage that was consumed last: its operand tiles
    // start at `epi_a` and `epi_b`.
    constexpr bool kStagedEpilogue = Cfg::WTN >= 32;
    [[maybe_unused]] uint8_t* epi_a = nullptr;
    [[maybe_unused]] uint8_t* epi_b = nullptr;
    // The second pass is a copy of the code, not a trip round a loop: as a loop with a run-time count even a single pass ran
    // 10 % slower (the compiler keeps less of the main loop's state where it was).
    constexpr int kMaxPasses = kTwoHalves ? 2 : 1;
#pragma unroll
    for (int pass = 0; pass < kMaxPasses; ++pass) {
    if (kTwoHalves && pass >= num_passes) break;
    if constexpr (kGemmType == GemmType::GroupedContiguous) {
        rhs        = rhs_all + size_t(pass_group[pass]) * N * K;
        rhs_scales = rhs_scales_all + size_t(pass_group[pass]) * NUM_N_BLOCKS * NUM_K_BLOCKS;
        rsrc_b     = make_rsrc(rhs, uint32_t(N) * K);
        if (pass) __syncthreads();        // every wave has read the last k-tile of the previous pass
        if constexpr (kTwoHalves) {
            const bool half_pass = num_passes == 2;
            rsrc_a_half[0] = half_pass && pass_lo[pass] != m0 ? rsrc_none : rsrc_a;
            rsrc_a_half[1] = half_pass && pass_hi[pass] == m0 + 128 ? rsrc_none : rsrc_a;
        }
    }
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    if constexpr (STAGES == 2) {
    uint8_t* const lds_a0 = two_stages.a0;
    uint8_t* const lds_b0 = two_stages.b0;
    uint8_t* const lds_a1 = two_stages.a1;
    uint8_t* const lds_b1 = two_stages.b1;
    stage_a.issue(rsrc_a, lds_a0, 0, wave);
    stage_b.issue(rsrc_b, lds_b0, 0, wave);
    load_scales(0);
    // A pass over one 128-row half of a 256-row tile: the waves whose slabs lie in the other half have nothing to multiply.
    // They run a loop of their own with the same barriers and their share of the copies, which leaves the matrix cores half
    // a tile per k-tile (a SIMD holds one wave of either half).
    bool other_half = false;
    if constexpr (kTwoHalves) {
        static_assert(128 % Cfg::WTM == 0, "a wave's slab lies in one half of the tile");
        other_half = num_passes == 2 && (m_slab < pass_lo[pass] || m_slab >= pass_hi[pass]);
    }
    if (kTwoHalves && other_half) {
        auto copy_step = [&](int kb, uint8_t* a_nxt, uint8_t* b_nxt) {
            wait_for_copies();
            __syncthreads();
#pragma unroll
            for (int d = 0; d < NUM_COPIES; ++d) {
                if (d < StA::PASSES) stage_a.issue_pass(rsrc_a_half[d * 2 / StA::PASSES], a_nxt, (kb + 1) * kRowBytes, wave, d);
                else stage_b.issue_pass(rsrc_b, b_nxt, (kb + 1) * kRowBytes, wave, d - StA::PASSES);
            }
        };
        for (int kb = 0; kb + 1 < NUM_K_BLOCKS; kb += 2) {
            copy_step(kb, lds_a1, lds_b1);
            copy_step(kb + 1, lds_a0, lds_b0);
        }
        if (NUM_K_BLOCKS % 2 == 1) copy_step(NUM_K_BLOCKS - 1, lds_a1, lds_b1);
    } else {
        for (int kb = 0; kb + 1 < NUM_K_BLOCKS; kb += 2) {
            k_step(kb, lds_a0, lds_b0, lds_a1, lds_b1);
            k_step(kb + 1, lds_a1, lds_b1, lds_a0, lds_b0);
        }
        if (NUM_K_BLOCKS % 2 == 1) k_step(NUM_K_BLOCKS - 1, lds_a0, lds_b0, lds_a1, lds_b1);
    }
    epi_a = (NUM_K_BLOCKS % 2 == 1) ? lds_a0 : lds_a1;
    epi_b = (NUM_K_BLOCKS % 2 == 1) ? lds_b0 : lds_b1;
    } else {
    // Ring of STAGES stages, STAGES - 1 k-tiles in flight: what a small tile needs when the problem is bound by
    // streaming its operands and one k-tile of prefetch cannot cover the memory latency. Every wave issues the same
    // number of copies for every k-tile (OPS), in the same order, so "k-tile kb has landed" is "at most
    // (STAGES - 2) * OPS of my copies are outstanding". The activation scales of a k-tile travel through the stage as well (a register load between the
    // copies would make the in-order counter wait for every older copy): every wave copies one 64-row part of them
    // with one full-width instruction; waves that share a part write the same bytes twice.
    constexpr int STAGE_BYTES = Cfg::RING_STAGE_BYTES, A_BYTES = Cfg::LDS_ROWS_A * kRowBytes, TILE_BYTES = A_BYTES + Cfg::LDS_ROWS_B * kRowBytes;
    constexpr int OPS = StA::PASSES + StB::PASSES + 1, SCALE_PARTS = BLOCK_M >= 64 ? BLOCK_M / 64 : 1;
    static_assert(Cfg::RING_CAPABLE && (fp8_ring_group(BLOCK_M, BLOCK_N, STAGES) > 1 || (STAGES - 2) * OPS <= 63) && STAGES * STAGE_BYTES <= 160 * 1024);
    uint8_t* ring = ring_lds;
    if constexpr (!EXTERNAL_RING) {
        __shared__ __attribute__((aligned(1024))) uint8_t own_ring[STAGES * STAGE_BYTES];
        ring = own_ring;
    }
    const uint32_t scale_voff = uint32_t(m0 + lane) * sa_stride_m * 4;
    auto issue_op = [&](int d, int kb, uint8_t* stage) {
        const bool live = kb < kb_hi;
        if (d < StA::PASSES) stage_a.issue_pass(live ? rsrc_a : rsrc_none, stage, kb * kRowBytes, wave, d);
        else if (d < StA::PASSES + StB::PASSES) stage_b.issue_pass(live ? rsrc_b : rsrc_none, stage + A_BYTES, kb * kRowBytes, wave, d - StA::PASSES);
        else {
            const int part = wave % SCALE_PARTS;                    // rows m0 + 64 * part + lane
            __builtin_amdgcn_raw_ptr_buffer_load_lds(live ? rsrc_sa : rsrc_none, YAN_LDS_PTR(stage + TILE_BYTES + part * 256), 4,
                                                     scale_voff, (kb * sa_stride_k + part * 64 * sa_stride_m) * 4, 0, 0);
        }
    };
    // Tiles of one or two atoms per wave (the decode shapes: 16 or 32 weight rows per workgroup) have almost nothing to
    // compute per k-tile, and a loop that meets at a barrier for every k-tile is bound by that chain of waits: barrier,
    // fragment reads, one MFMA, its fold, 56 times over. They consume the ring G k-tiles at a time instead: one
    // barrier, the fragments of G k-tiles, G independent MFMAs, G folds; the copies of the G k-tiles that go where the
    // previous group was start right after the barrier, so STAGES - 2G to STAGES - G k-tiles are in flight.
    constexpr int G = fp8_ring_group(BLOCK_M, BLOCK_N, STAGES);
    if constexpr (G > 1) {
    // Eight waves share the copies of a k-tile: operation o = slot * 8 + wave is the o-th 8-row group of the stage
    // (activation rows first, then weight rows: the two tiles lie back to back) or, past the last group, the copy of
    // the activation scales (which several waves may repeat: same bytes).
    constexpr int GA = BLOCK_M / 8, GROUPS_AB = (BLOCK_M + BLOCK_N) / 8, SLOTS = ceil_div(GROUPS_AB + 1, LW);
    static_assert(LW == 8 && NW == 4 && A_BYTES == GA * 8 * kRowBytes && TILE_BYTES == GROUPS_AB * 8 * kRowBytes && SCALE_PARTS == 1);
    static_assert(Cfg::UNIFORM_SCALE_B && NB == 1 && (STAGES - 2 * G) * SLOTS <= 63);
    uint32_t slot_voff[SLOTS];
#pragma unroll
    for (int sl = 0; sl < SLOTS; ++sl) {
        const int o = sl * LW + wave, sub = lane >> 3, chunk = (lane & 7) ^ sub ^ (o & 1);      // GA is even: o and its group in B have the same parity
        const int row = (o < GA ? m0 + o * 8 : n0 + (o - GA) * 8) + sub;
        slot_voff[sl] = uint32_t(row) * K + chunk * kChunk;
    }
    auto issue_slot = [&](int sl, int kb, uint8_t* stage) {
        const int o = sl * LW + wave;
        const bool live = kb < kb_hi;
        // which kind of operation a slot holds is known at compile time unless the slot straddles two kinds
        const bool data = sl * LW + LW - 1 < GROUPS_AB || (sl * LW < GROUPS_AB && o < GROUPS_AB);
        const bool in_a = sl * LW + LW - 1 < GA || (sl * LW < GA && o < GA);
        if (data) {
            if (in_a) __builtin_amdgcn_raw_ptr_buffer_load_lds(live ? rsrc_a : rsrc_none, YAN_LDS_PTR(stage + o * 8 * kRowBytes), kChunk, slot_voff[sl], kb * kRowBytes, 0, 0);
            else __builtin_amdgcn_raw_ptr_buffer_load_lds(live ? rsrc_b : rsrc_none, YAN_LDS_PTR(stage + o * 8 * kRowBytes), kChunk, slot_voff[sl], kb * kRowBytes, 0, 0);
        } else {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(live ? rsrc_sa : rsrc_none, YAN_LDS_PTR(stage + TILE_BYTES), 4, scale_voff, kb * sa_stride_k * 4, 0, 0);
        }
    };
#pragma unroll
    for (int t = 0; t < STAGES - G; ++t)
#pragma unroll
        for (int sl = 0; sl < SLOTS; ++sl) issue_slot(sl, kb_lo + t, ring + t * STAGE_BYTES);
    int base = 0;          // ring position of the group's first k-tile; STAGES is a multiple of G, groups never wrap
    for (int kb0 = kb_lo; kb0 < kb_hi; kb0 += G) {
        __builtin_amdgcn_s_waitcnt(waitcnt_imm((STAGES - 2 * G) * SLOTS, kNoWaitLgkm));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // every wave has left the previous group: its stages take k-tiles kb0 + STAGES - G .. kb0 + STAGES - 1 (past the
        // last k-tile these move bytes nobody reads; they are issued all the same, the waits count instructions)
        const int prev = base == 0 ? STAGES - G : base - G;
#pragma unroll
        for (int t = 0; t < G; ++t)
#pragma unroll
            for (int sl = 0; sl < SLOTS; ++sl) issue_slot(sl, kb0 + STAGES - G + t, ring + (prev + t) * STAGE_BYTES);
        if (wave < NW) {
        float sb_grp[G];
#pragma unroll
        for (int t = 0; t < G; ++t)
            sb_grp[t] = rhs_scales[min(base_blk, NUM_N_BLOCKS - 1) * NUM_K_BLOCKS + min(kb0 + t, NUM_K_BLOCKS - 1)];
        f32x4 part[G][TN][TM];
        float s_grp[G][TM];
#pragma unroll
        for (int t = 0; t < G; ++t) {
            const uint8_t* cur = ring + (base + t) * STAGE_BYTES;
            const uint8_t* pa = cur + wm * Cfg::WTM * kRowBytes;
            const uint8_t* pb = cur + A_BYTES + wn * Cfg::WTN * kRowBytes;
            const float* my_scales = reinterpret_cast<const float*>(cur + TILE_BYTES) + wm * Cfg::WTM + col;
            i32x8 mf[TM], nf[TN];
#pragma unroll
            for (int j = 0; j < TM; ++j) { mf[j] = read_frag(pa + j * 16 * kRowBytes); s_grp[t][j] = my_scales[j * 16] * sb_grp[t]; }
#pragma unroll
            for (int i = 0; i < TN; ++i) nf[i] = read_frag(pb + i * 16 * kRowBytes);
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int j = 0; j < TM; ++j) part[t][i][j] = Atom::mma(nf[i], mf[j], f32x4{0.f, 0.f, 0.f, 0.f});
        }
#pragma unroll
        for (int t = 0; t < G; ++t) {
            if (kb0 + t < kb_hi) {          // wave-uniform; nothing was copied for k-tiles past the end
#pragma unroll
                for (int i = 0; i < TN; ++i)
#pragma unroll
                    for (int j = 0; j < TM; ++j)
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[i][j][r] = __builtin_fmaf(part[t][i][j][r], s_grp[t][j], acc[i][j][r]);
            }
        }
        }
        base = base + G == STAGES ? 0 : base + G;
    }
    // the first stage of the group that was consumed last: no copy is on its way into it
    epi_a = ring + (base == 0 ? STAGES - G : base - G) * STAGE_BYTES;
    epi_b = epi_a + A_BYTES;
    } else {
#pragma unroll
    for (int t = 0; t < STAGES - 1; ++t)
#pragma unroll
        for (int d = 0; d < OPS; ++d) issue_op(d, kb_lo + t, ring + t * STAGE_BYTES);
    load_weight_scales(min(kb_lo, NUM_K_BLOCKS - 1));
    int st = 0;
    for (int kb = kb_lo; kb < kb_hi; ++kb) {
#pragma unroll
        for (int b = 0; b < NB; ++b) sb_cur[b] = sb_next[b];
        __builtin_amdgcn_s_waitcnt(waitcnt_imm((STAGES - 2) * OPS, kNoWaitLgkm));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        load_weight_scales(min(kb + 1, NUM_K_BLOCKS - 1));
        const uint8_t* cur = ring + st * STAGE_BYTES;
        const int st_nxt = st + STAGES - 1 >= STAGES ? st - 1 : st + STAGES - 1;
        uint8_t* nxt = ring + st_nxt * STAGE_BYTES;
        const float* my_scales = reinterpret_cast<const float*>(cur + TILE_BYTES) + wm * Cfg::WTM + col;
#pragma unroll
        for (int j = 0; j < TM; ++j) sa_cur[j] = my_scales[j * 16];
        compute_tile(cur, cur + A_BYTES, sa_cur, sb_cur, [&](int row) {
#pragma unroll
            for (int d = 0; d < OPS; ++d)
                if (d * SPREAD_ROWS / OPS == row) issue_op(d, kb + STAGES - 1, nxt);
        });
        st = st + 1 == STAGES ? 0 : st + 1;
    }
    epi_a = ring + (st == 0 ? STAGES - 1 : st - 1) * STAGE_BYTES;
    epi_b = epi_a + A_BYTES;
    }
    }

    // Epilogue (fp8_store_slab): slabs of 32 columns or more turn round through the LDS stage that was consumed last (the
    // only one no copy is on its way into) when the rows of the output are 16-byte aligned.
    // An output larger than the L2s together (8 x 4 MB) is stored with the non-temporal hint: kept in L2 it pushes out
    // the operand panels the other workgroups of the XCD are about to read.
    bool staged = false;
    if constexpr (kStagedEpilogue) staged = (N % 8) == 0;
    const bool stream_out = size_t(m) * N * 2 * (kGemmType == GemmType::GroupedMasked ? num_groups : 1) > (size_t(32) << 20);
    const __amdgpu_buffer_rsrc_t rsrc_out = make_out_rsrc(out + size_t(m0) * N + n0);
    if (staged) {
        constexpr int REGION = 16 * (Cfg::WTN * 2 + 16);
        static_assert(!kStagedEpilogue || ((NW / 2) * REGION <= Cfg::LDS_ROWS_A * kRowBytes && (NW / 2) * REGION <= Cfg::LDS_ROWS_B * kRowBytes));
        // every wave has read the last k-tile (a bare barrier: __syncthreads() would also wait for the copies still
        // on their way into the other stages, which nobody will read)
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoWaitVm, 0));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (LW > NW && wave >= NW) return;          // waves that only copy
        // Everything the epilogue derives from the lane number is derived behind an opaque copy of it: the main loop
        // has no registers to spare for addresses computed ahead of time.
        int lane_late = lane;
        asm volatile("" : "+v"(lane_late));
        if constexpr (SPLIT_K > 1)
            if (!fp8_meet_partials<SPLIT_K, NW, TN, TM>(acc, partials, counters, tile_slot, split, wave, lane_late)) return;
        uint8_t* region = (wave < NW / 2 ? epi_a : epi_b) + (wave % (NW / 2)) * REGION;
        fp8_store_slab<Cfg, kStagedEpilogue>(acc, region, rsrc_out, m_slab, n_slab, m0, n0, pass_lo[pass], pass_hi[pass], N, stream_out, lane_late);
    } else {
        if (LW > NW && wave >= NW) return;              // waves that only copy
        if constexpr (SPLIT_K > 1)
            if (!fp8_meet_partials<SPLIT_K, NW, TN, TM>(acc, partials, counters, tile_slot, split, wave, lane)) return;
        fp8_store_slab<Cfg, false>(acc, nullptr, rsrc_out, m_slab, n_slab, m0, n0, pass_lo[pass], pass_hi[pass], N, stream_out, lane);
    }
    }   // pass
}

// Whether a problem runs the persistent walk below: the plain GEMM on two LDS stages with an even number of k-tiles
// (every tile then starts in stage 0).
template <int STAGES, GemmType kGemmType>
__host__ __device__ constexpr bool fp8_walks(int k) {
    return STAGES == 2 && kGemmType == GemmType::Normal && (k / 128) % 2 == 0;
}

// The plain GEMM on two LDS stages as a persistent walk: workgroup b takes slots b, b + gridDim.x, ... (the launcher
// starts one workgroup per CU, or as many as the caller's cap allows) and overlaps the seams between them. The copies of
// the next tile's first k-tile and its first scales start during the last k-tile of the current one, every wave waits
// for them in front of the epilogue, and the output stores drain while the next tile's first k-tile is being
// multiplied. With a workgroup per tile every tile pays for its first loads, its store drain and a workgroup launch:
// 4096 x 7168 x 7168 runs 1.5 % faster this way, 4096 x 24576 x 1536 5 %, 4096 x 32768 x 512 15 %. Same bits: the sum
// over K is formed in the same order.
// What a wave needs to know of a tile is wave-uniform: the per-lane parts of every address (the lane's row within a copy
// pass, its row within the slab) do not depend on the tile, and the tile's first row rides in the scalar offset.
template <int SHAPE_N, int SHAPE_K, int BLOCK_M, int BLOCK_N>
__device__ __forceinline__ void
fp8_gemm_walk(const uint8_t* __restrict__ lhs, const float* __restrict__ lhs_scales,
              const uint8_t* __restrict__ rhs, const float* __restrict__ rhs_scales,
              __bf16* __restrict__ out, int m, int n_rt, int k_rt, int sa_stride_m, int sa_stride_k, int num_slots, Fp8TwoStages two_stages) {
    using Cfg = Fp8TileConfig<BLOCK_M, BLOCK_N>;
    constexpr int NW = Cfg::NUM_WAVES, TN = Cfg::WTN / 16, TM = Cfg::WTM / 16, NB = Cfg::SCALE_B_PER_SLAB;
    // SHAPE_N / SHAPE_K == 0 selects the run-time sizes (ahead-of-time library); the JIT bakes them in.
    const int N = SHAPE_N ? SHAPE_N : n_rt, K = SHAPE_K ? SHAPE_K : k_rt;
    const int NUM_K_BLOCKS = K / 128, NUM_N_BLOCKS = ceil_div(N, 128);          // NUM_K_BLOCKS is even: the caller checked
    static_assert(Cfg::WTN >= 32);
    using StA = TileStager<BLOCK_M, NW>;
    using StB = TileStager<BLOCK_N, NW>;
    constexpr int NUM_COPIES = StA::PASSES + StB::PASSES, SPREAD_ROWS = TN >= 2 ? TN / 2 : 1;

    const XcdTileScheduler<> sched(m, N, BLOCK_M, BLOCK_N, (long long)K);
    const int lane = get_lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const int wn = wave % Cfg::WAVES_N, wm = wave / Cfg::WAVES_N;
    const int g = lane / 16, col = lane % 16;

    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(lhs, uint32_t(m) * K);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(rhs, uint32_t(N) * K);
    const uint32_t sa_bytes = (uint32_t(m - 1) * sa_stride_m + uint32_t(NUM_K_BLOCKS - 1) * sa_stride_k + 1) * 4;
    const __amdgpu_buffer_rsrc_t rsrc_sa = make_rsrc(lhs_scales, sa_bytes);
    // Output stores are plain here at every size: they drain while the next tile's first k-tile is multiplied, and
    // since loads and stores of a wave complete in order, stores that the L2 takes in at once free the loads behind
    // them sooner than non-temporal ones (4096 x 24576 x 1536: 145 -> 138 us; 8192 x 7168 x 7168: 339 -> 336 us).
    // The one-tile-per-slot kernel above is the other way round (4 groups of 4096 x 4096 x 7168: 439 us non-temporal,
    // 506 us plain).
    constexpr bool stream_out = false;

    struct TileIo {
        int m0, n0;
        int base_blk, rows_in_first_block;      // weight-scale blocks of the slab
        bool valid;
    };
    auto open_tile = [&](int slot) {
        TileIo t;
        const TileCoord coord = slot < num_slots ? sched.tile_of(slot) : TileCoord{0, 0, false};
        t.valid = coord.valid;
        // no tile: activation rows past the matrix (its copies move zeros, its scale loads return zeros), weight tile 0
        t.m0 = coord.valid ? coord.m_idx * BLOCK_M : sched.tiles_m * BLOCK_M;
        t.n0 = coord.n_idx * BLOCK_N;
        const int n_slab = t.n0 + wn * Cfg::WTN;
        t.base_blk = n_slab / 128;
        t.rows_in_first_block = (128 - (n_slab & 127)) / 16;
        return t;
    };
    StA stage_a;
    StB stage_b;
    stage_a.init(0, K, wave, lane);
    stage_b.init(0, K, wave, lane);
    const uint32_t sa_voff = uint32_t(wm * Cfg::WTM + col) * sa_stride_m * 4;
    const int off0 = frag_offset<16>(lane, 2 * g), off1 = frag_offset<16>(lane, 2 * g + 1);

    f32x4 acc[TN][TM];
    float sa_next[TM], sb_next[NB], sa_cur[TM], sb_cur[NB];
    auto load_scales = [&](const TileIo& t, int kb) {
#pragma unroll
        for (int j = 0; j < TM; ++j)
            sa_next[j] = buffer_load_f32(rsrc_sa, sa_voff, (kb * sa_stride_k + (t.m0 + j * 16) * sa_stride_m) * 4);
#pragma unroll
        for (int b = 0; b < NB; ++b) sb_next[b] = rhs_scales[min(t.base_blk + b, NUM_N_BLOCKS - 1) * NUM_K_BLOCKS + kb];
    };

    uint8_t* const lds_a0 = two_stages.a0;
    uint8_t* const lds_b0 = two_stages.b0;
    uint8_t* const lds_a1 = two_stages.a1;
    uint8_t* const lds_b1 = two_stages.b1;

    // One k-tile of tile `t`, staged in (a_cur, b_cur) and known to have landed when `landed`; meanwhile the copies of
    // k-tile `kb_src` of tile `src` go into (a_nxt, b_nxt) and its scales into registers (`src` is `t` itself, or the
    // next tile during the last k-tile).
    auto k_step = [&](const TileIo& t, const uint8_t* a_cur, const uint8_t* b_cur, uint8_t* a_nxt, uint8_t* b_nxt,
                      const TileIo& src, int kb_src, bool landed) {
        const int a_byte0 = src.m0 * K + kb_src * kRowBytes, b_byte0 = src.n0 * K + kb_src * kRowBytes;
#pragma unroll
        for (int j = 0; j < TM; ++j) sa_cur[j] = sa_next[j];
#pragma unroll
        for (int b = 0; b < NB; ++b) sb_cur[b] = sb_next[b];
        if (!landed) {
            wait_for_copies();
            __syncthreads();
        }
        load_scales(src, kb_src);
        fp8_compute_k_tile<Cfg>(acc, a_cur + wm * Cfg::WTM * kRowBytes, b_cur + wn * Cfg::WTN * kRowBytes, sa_cur, sb_cur,
                                t.rows_in_first_block, off0, off1, [&](int row) {
#pragma unroll
            for (int d = 0; d < NUM_COPIES; ++d) {
                if (d * SPREAD_ROWS / NUM_COPIES != row) continue;
                if (d < StA::PASSES) stage_a.issue_pass(rsrc_a, a_nxt, a_byte0, wave, d);
                else stage_b.issue_pass(rsrc_b, b_nxt, b_byte0, wave, d - StA::PASSES);
            }
        });
    };

    // The next slot of this workgroup's walk that holds a tile. Under a cap that is not a multiple of the 8 XCDs a walk
    // crosses the XCDs' ranges, and an empty slot at the end of one range can be followed by a tile of another.
    auto seek = [&](int slot) {
        while (slot < num_slots && !sched.tile_of(slot).valid) slot += gridDim.x;
        return slot;
    };
    int slot = seek(blockIdx.x);
    TileIo cur = open_tile(slot);
    if (!cur.valid) return;
    stage_a.issue(rsrc_a, lds_a0, cur.m0 * K, wave);
    stage_b.issue(rsrc_b, lds_b0, cur.n0 * K, wave);
    load_scales(cur, 0);
    wait_for_copies();
    __syncthreads();
    while (true) {
        slot = seek(slot + gridDim.x);
        const TileIo nxt = open_tile(slot);
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        // k-tile 0 has landed for every wave: the barrier in front of the loop, or the one in front of the last epilogue
        k_step(cur, lds_a0, lds_b0, lds_a1, lds_b1, cur, 1, true);
        for (int kb = 1; kb + 2 < NUM_K_BLOCKS; kb += 2) {
            k_step(cur, lds_a1, lds_b1, lds_a0, lds_b0, cur, kb + 1, false);
            k_step(cur, lds_a0, lds_b0, lds_a1, lds_b1, cur, kb + 2, false);
        }
        // the last k-tile, in stage 1; stage 0 takes the first k-tile of the next tile
        k_step(cur, lds_a1, lds_b1, lds_a0, lds_b0, nxt, 0, false);
        // the sums are complete here: without this the compiler moves the last folds down into the epilogue, next to their
        // first use, and parks the partial sums they wait for in scratch memory
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j) asm volatile("" : "+v"(acc[i][j]));

        // every wave has read the last k-tile and the next tile's first k-tile has landed; then the epilogue through stage 1
        wait_for_copies();
        __syncthreads();
        {
            constexpr int REGION = 16 * (Cfg::WTN * 2 + 16);
            static_assert((NW / 2) * REGION <= Cfg::LDS_ROWS_A * kRowBytes && (NW / 2) * REGION <= Cfg::LDS_ROWS_B * kRowBytes);
            const __amdgpu_buffer_rsrc_t rsrc_out = make_out_rsrc(out + size_t(cur.m0) * N + cur.n0);
            int lane_late = lane;
            asm volatile("" : "+v"(lane_late));
            uint8_t* region = (wave < NW / 2 ? lds_a1 : lds_b1) + (wave % (NW / 2)) * REGION;
            if ((N % 8) == 0)
                fp8_store_slab<Cfg, true>(acc, region, rsrc_out, cur.m0 + wm * Cfg::WTM, cur.n0 + wn * Cfg::WTN, cur.m0, cur.n0,
                                          0, m, N, stream_out, lane_late);
            else
                fp8_store_slab<Cfg, false>(acc, region, rsrc_out, cur.m0 + wm * Cfg::WTM, cur.n0 + wn * Cfg::WTN, cur.m0, cur.n0,
                                           0, m, N, stream_out, lane_late);
        }
        if (!nxt.valid) break;
        cur = nxt;
        // the next tile's second k-tile is copied into the stage the epilogue went through: every wave has to be out of it
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoWaitVm, 0));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    }
}

// Workgroup b runs slots b, b + gridDim.x, ...: the persistent walk above where it applies; otherwise exactly one slot
// when the launcher starts a workgroup per slot, and a plain loop over several when the caller caps the number of compute
// units (the reference's persistent kernel under `num_sms`,
// yan/include/gemm/fp8_gemm.cuh:40, scheduler.cuh:39-58). Between two tiles every wave must have left the epilogue of
// the first (which reads the LDS stage the second one's first copies go into).
template <int SHAPE_N, int SHAPE_K, int BLOCK_M, int BLOCK_N, GemmType kGemmType = GemmType::Normal, int STAGES = 2>
__global__ void __launch_bounds__((fp8_launch_waves(BLOCK_M, BLOCK_N, STAGES) * kWaveSize))
fp8_gemm_kernel(const uint8_t* __restrict__ lhs, const float* __restrict__ lhs_scales,
                const uint8_t* __restrict__ rhs, const float* __restrict__ rhs_scales,
                __bf16* __restrict__ out, int m, int n_rt, int k_rt, int sa_stride_m, int sa_stride_k,
                const int* __restrict__ grouped_layout, int sa_stride_g, int num_slots, int num_groups, int expected_m) {
    Fp8TwoStages two_stages = {nullptr, nullptr, nullptr, nullptr};
    if constexpr (STAGES == 2) {
        using Cfg = Fp8TileConfig<BLOCK_M, BLOCK_N>;
        __shared__ __attribute__((aligned(1024))) uint8_t lds_a0[Cfg::LDS_ROWS_A * kRowBytes];
        __shared__ __attribute__((aligned(1024))) uint8_t lds_b0[Cfg::LDS_ROWS_B * kRowBytes];
        __shared__ __attribute__((aligned(1024))) uint8_t lds_a1[Cfg::LDS_ROWS_A * kRowBytes];
        __shared__ __attribute__((aligned(1024))) uint8_t lds_b1[Cfg::LDS_ROWS_B * kRowBytes];
        two_stages = {lds_a0, lds_b0, lds_a1, lds_b1};
    }
    if constexpr (fp8_walks<STAGES, kGemmType>(SHAPE_K)) {
        if (SHAPE_K != 0 || fp8_walks<STAGES, kGemmType>(k_rt)) {
            fp8_gemm_walk<SHAPE_N, SHAPE_K, BLOCK_M, BLOCK_N>(lhs, lhs_scales, rhs, rhs_scales, out, m, n_rt, k_rt, sa_stride_m, sa_stride_k,
                                                              num_slots, two_stages);
            return;
        }
    }
    // A workgroup per slot (no cap): the tile without a loop around it. Inside the loop below the same code runs 2 to 14 %
    // slower on the ring tiles even for a single trip (64 x 7168 x 2048 on 64 x 32 tiles: 6.0 against 5.2 us).
    if (int(gridDim.x) >= num_slots) {
        fp8_gemm_tile<SHAPE_N, SHAPE_K, BLOCK_M, BLOCK_N, kGemmType, STAGES>(lhs, lhs_scales, rhs, rhs_scales, out, m, n_rt, k_rt,
                                                                             sa_stride_m, sa_stride_k, grouped_layout, sa_stride_g,
                                                                             int(blockIdx.x), num_groups, expected_m, two_stages);
        return;
    }
    for (int slot = blockIdx.x; slot < num_slots; slot += gridDim.x) {
        fp8_gemm_tile<SHAPE_N, SHAPE_K, BLOCK_M, BLOCK_N, kGemmType, STAGES>(lhs, lhs_scales, rhs, rhs_scales, out, m, n_rt, k_rt,
                                                                             sa_stride_m, sa_stride_k, grouped_layout, sa_stride_g,
                                                                             slot, num_groups, expected_m, two_stages);
        if (slot + int(gridDim.x) < num_slots) __syncthreads();
    }
}

// Contiguous groups on 256-row tiles, with what a tile row that holds two groups costs decided on the device. Which rows
// those are is in the caller's layout; the host cannot look. A 256-row tile whose halves belong to two groups makes two
// passes over K and takes about 1.7 tile times (fp8_gemm_tile's two-pass path); as two 128 x BLOCK_N tiles on the ring its
// halves take 1.2 to 1.3 together and can go to two workgroups, but a launch that ends on half tiles ends raggedly.
// This kernel holds both tiles over one pool of LDS; every workgroup counts the tile rows that hold two groups (two
// loads per lane and a ballot: `two` of `rows`) and all number the slots alike, one of three ways (measured with
// 4096 x 7168 weights; all three give the same bits):
//   * two * 20 < rows (long groups, or every boundary on a multiple of 256 rows): 256-row tiles throughout, the two-pass
//     tiles first (ContiguousSlots). 16 groups of 512 rows: 225 us against 264 on 128 x 256 tiles; groups of 1920 to 2176 rows
//     with one such row in 32: 223 against 238 for the next way;
//   * up to a quarter of the rows: the whole 256-row tiles of the other rows first, in band order dealt to the XCDs in
//     patches, then the half tiles of the two-group rows, the shorter jobs, which fill the end of the launch. 8 groups of
//     896 and 1152 rows: 230 us against 251 with two-pass tiles; 16 of 384 and 640: 271 against 284 on 128-row tiles;
//   * more than a quarter (groups of less than two tile rows: a 256-row tile has no neighbour to share its weight panel
//     with): 128 x BLOCK_N tiles throughout. 16 groups of 384 rows: 205 us against 216 for the second way.
// It is launched with eight slots more than the 128-row tiling has, which covers every case; workgroups beyond the last
// slot leave at once.
template <int SHAPE_N, int SHAPE_K, int BLOCK_N>
__global__ void __launch_bounds__(8 * kWaveSize)
fp8_gemm_contiguous_rows_kernel(const uint8_t* __restrict__ lhs, const float* __restrict__ lhs_scales,
                                const uint8_t* __restrict__ rhs, const float* __restrict__ rhs_scales,
                                __bf16* __restrict__ out, int m, int n_rt, int k_rt, int sa_stride_m, int sa_stride_k,
                                const int* __restrict__ grouped_layout, int num_groups) {
    using Tall = Fp8TileConfig<256, BLOCK_N>;
    using Flat = Fp8TileConfig<128, BLOCK_N>;
    constexpr int FLAT_STAGES = Flat::MAX_RING_STAGES;
    constexpr int TALL_BYTES = 2 * (Tall::LDS_ROWS_A + Tall::LDS_ROWS_B) * kRowBytes, FLAT_BYTES = FLAT_STAGES * Flat::RING_STAGE_BYTES;
    static_assert(FLAT_STAGES >= 3 && fp8_launch_waves(256, BLOCK_N, 2) == 8 && fp8_launch_waves(128, BLOCK_N, FLAT_STAGES) == 8);
    __shared__ __attribute__((aligned(1024))) uint8_t pool[TALL_BYTES > FLAT_BYTES ? TALL_BYTES : FLAT_BYTES];
    uint8_t* const a0 = pool;
    uint8_t* const b0 = a0 + Tall::LDS_ROWS_A * kRowBytes;
    uint8_t* const a1 = b0 + Tall::LDS_ROWS_B * kRowBytes;
    uint8_t* const b1 = a1 + Tall::LDS_ROWS_A * kRowBytes;
    const int N = SHAPE_N ? SHAPE_N : n_rt;
    const int lane = get_lane_id();
    const int tall_rows = ceil_div(m, 256), tiles_n = ceil_div(N, BLOCK_N);
    const int two_group_rows = count_two_group_rows(grouped_layout, m, tall_rows, lane);
    // tile (row, column) of the 256-row / 128-row grid
    auto tall_tile = [&](int row, int n_idx) {
        fp8_gemm_tile<SHAPE_N, SHAPE_K, 256, BLOCK_N, GemmType::GroupedContiguous, 2, 1, false, true>(
            lhs, lhs_scales, rhs, rhs_scales, out, m, n_rt, k_rt, sa_stride_m, sa_stride_k, grouped_layout, 0, row * tiles_n + n_idx, num_groups, 0,
            Fp8TwoStages{a0, b0, a1, b1});
    };
    auto flat_tile = [&](int row, int n_idx) {
        fp8_gemm_tile<SHAPE_N, SHAPE_K, 128, BLOCK_N, GemmType::GroupedContiguous, FLAT_STAGES, 1, true, true>(
            lhs, lhs_scales, rhs, rhs_scales, out, m, n_rt, k_rt, sa_stride_m, sa_stride_k, grouped_layout, 0, row * tiles_n + n_idx, num_groups, 0,
            Fp8TwoStages{nullptr, nullptr, nullptr, nullptr}, nullptr, nullptr, pool);
    };
    const int mode = two_group_rows * 20 < tall_rows ? 0 : (two_group_rows * 4 <= tall_rows ? 1 : 2);
    // the rows that hold one group (or one group and padding), as a grid of their own (mode 1)
    XcdTileScheduler<> whole((tall_rows - two_group_rows) * 256, N, 256, BLOCK_N);
    whole.fit_bands_to_groups((tall_rows - two_group_rows) / max(num_groups, 1));
    XcdTileScheduler<> flat(m, N, 128, BLOCK_N);
    flat.fit_bands_to_groups(flat.tiles_m / max(num_groups, 1));
    const ContiguousSlots two_pass_first(m, N, 256, BLOCK_N, num_groups, two_group_rows);
    const int whole_slots = whole.grid_size();
    const int slots = mode == 0 ? int(ContiguousSlots::num_slots(m, N, 256, BLOCK_N))
                                : (mode == 1 ? whole_slots + 2 * two_group_rows * tiles_n : flat.grid_size());
    // Either tile's code appears once (the compiler gives each copy of it its own registers, and four copies spill).
    auto run_slot = [&](int slot) {
        TileCoord t{0, 0, false};       // of the 256-row grid, or of the 128-row grid when `half_tile`
        bool half_tile = false;
        if (mode == 0) {
            t = two_pass_first.tile_of(slot);
            if (t.valid && two_group_rows) t.m_idx = contiguous_row_at(grouped_layout, m, tall_rows, two_group_rows, t.m_idx, lane);
        } else if (mode == 2) {
            t = flat.tile_of(slot);
            half_tile = true;
        } else if (slot < whole_slots) {
            t = whole.dealt_band_tile_of(slot);
            if (t.valid) t.m_idx = contiguous_row_at(grouped_layout, m, tall_rows, two_group_rows, two_group_rows + t.m_idx, lane);
        } else {
            const int h = slot - whole_slots, within = h % (2 * tiles_n);
            t = TileCoord{2 * contiguous_row_at(grouped_layout, m, tall_rows, two_group_rows, h / (2 * tiles_n), lane) + (within & 1), within / 2, true};
            half_tile = true;
        }
        if (!t.valid) return;
        if (half_tile) flat_tile(t.m_idx, t.n_idx);
        else tall_tile(t.m_idx, t.n_idx);
    };
    const int grid = gridDim.x;
    // a workgroup per slot (no cap): the tile without a loop around it
    if (grid >= slots) {
        if (int(blockIdx.x) < slots) run_slot(blockIdx.x);
        return;
    }
    for (int slot = blockIdx.x; slot < slots; slot += grid) {
        run_slot(slot);
        if (slot + grid < slots) __syncthreads();
    }
}

// The same tiles with K split SPLIT_K ways: launch slot s is part s % SPLIT_K of tile slot s / SPLIT_K.
template <int SHAPE_N, int SHAPE_K, int BLOCK_M, int BLOCK_N, int STAGES, int SPLIT_K>
__global__ void __launch_bounds__((fp8_launch_waves(BLOCK_M, BLOCK_N, STAGES) * kWaveSize))
fp8_gemm_split_k_kernel(const uint8_t* __restrict__ lhs, const float* __restrict__ lhs_scales,
                        const uint8_t* __restrict__ rhs, const float* __restrict__ rhs_scales,
                        __bf16* __restrict__ out, int m, int n_rt, int k_rt, int sa_stride_m, int sa_stride_k,
                        float* __restrict__ partials, unsigned* __restrict__ counters) {
    fp8_gemm_tile<SHAPE_N, SHAPE_K, BLOCK_M, BLOCK_N, GemmType::Normal, STAGES, SPLIT_K>(
        lhs, lhs_scales, rhs, rhs_scales, out, m, n_rt, k_rt, sa_stride_m, sa_stride_k, nullptr, 0, int(blockIdx.x), 1, 0,
        Fp8TwoStages{nullptr, nullptr, nullptr, nullptr}, partials, counters);
}

// Host side of the kernel, shaped after the class the reference's JIT template instantiates
// (yan/jit_kernels/gemm.py:20-30: Gemm<N, K, BLOCK_M, BLOCK_N, 128, 1, kNumStages, kNumTMAMulticast, Normal>::run).
// BLOCK_K is fixed at 128. kNumStages is the number of LDS stages: 2, or a ring of 3 .. Fp8TileConfig::MAX_RING_STAGES
// for the small tiles that support one. kNumTMAMulticast is accepted and unused (gfx950 has no multicast copy), as
// is `smem_size` (static LDS). `num_sms` caps the number of workgroups, as it sizes the reference's persistent grid
// (capped_grid in scheduler.hpp).
template <uint32_t SHAPE_N, uint32_t SHAPE_K, uint32_t BLOCK_M, uint32_t BLOCK_N, uint32_t BLOCK_K,
          uint32_t kNumGroups, uint32_t kNumStages, uint32_t kNumTMAMulticast, GemmType kGemmType>
class Gemm {
    static_assert(BLOCK_K == 128, "one k-tile is one 128-deep scale block");
    static_assert(kGemmType != GemmType::Normal || kNumGroups == 1, "a plain GEMM has one group");
    static_assert(kGemmType != GemmType::GroupedContiguous || 128 % BLOCK_M == 0 || BLOCK_M == 256, "contiguous groups are padded to 128 rows");

public:
    // lhs [m, K] e4m3 row-major; lhs_scales fp32, element (i, kb) at i * stride_m + kb * stride_k;
    // rhs [N, K] e4m3 row-major; rhs_scales fp32 [ceil(N/128), K/128] row-major; out [m, N] bf16 row-major.
    static hipError_t run(__hip_bfloat16* out, const void* lhs, const float* lhs_scales, int lhs_scales_stride_m,
                          int lhs_scales_stride_k, const void* rhs, const float* rhs_scales, int m,
                          hipStream_t stream, int num_sms, uint32_t smem_size) {
        static_assert(kGemmType == GemmType::Normal, "grouped layouts go through run_grouped");
        return run_sized(out, lhs, lhs_scales, lhs_scales_stride_m, lhs_scales_stride_k, rhs, rhs_scales, m,
                         int(SHAPE_N), int(SHAPE_K), stream, num_sms, smem_size);
    }

    // Grouped layouts (see the kernel's comment). `m` is the total number of rows (contiguous) or the rows
    // allotted to each group (masked); `grouped_layout` is a device array of m (contiguous) or num_groups (masked)
    // ints; `lhs_scales_stride_g` is used by the masked layout only, as is `expected_m` (the rows of a group that usually
    // exist; 0: all of them): it orders the slots, the result does not depend on it. n and k as in run_sized.
    static hipError_t run_grouped(__hip_bfloat16* out, const void* lhs, const float* lhs_scales, int lhs_scales_stride_m,
                                  int lhs_scales_stride_k, int lhs_scales_stride_g, const void* rhs, const float* rhs_scales,
                                  const int* grouped_layout, int num_groups, int m, int n, int k, hipStream_t stream,
                                  int num_sms = 0, int expected_m = 0) {
        static_assert(kGemmType != GemmType::Normal);
        if (m == 0 || n == 0 || num_groups == 0) return hipSuccess;
        if (m < 0 || n < 0 || k <= 0 || num_groups < 0 || (n % 4) != 0 || (k % 128) != 0) return hipErrorInvalidValue;
        if ((SHAPE_N && n != int(SHAPE_N)) || (SHAPE_K && k != int(SHAPE_K))) return hipErrorInvalidValue;
        if (kNumGroups > 1 && num_groups != int(kNumGroups)) return hipErrorInvalidValue;
        if (!out || !lhs || !lhs_scales || !rhs || !rhs_scales || !grouped_layout) return hipErrorInvalidValue;
        const uint64_t m_pad = uint64_t(ceil_div<uint32_t>(m, BLOCK_M)) * BLOCK_M, n_pad = uint64_t(ceil_div<uint32_t>(n, BLOCK_N)) * BLOCK_N;
        if (m_pad * k >= kOutOfRange || n_pad * k >= kOutOfRange) return hipErrorInvalidValue;
        // output stores address a tile with 32-bit byte offsets from its first element: BLOCK_M rows of n elements
        if (uint64_t(BLOCK_M) * n * 2 >= kOutOfRange) return hipErrorInvalidValue;
        using Cfg = Fp8TileConfig<BLOCK_M, BLOCK_N>;
        if (m_pad * num_groups >= kOutOfRange) return hipErrorInvalidValue;
        const XcdTileScheduler<> sched(m, n, BLOCK_M, BLOCK_N);
        const uint64_t slots = kGemmType == GemmType::GroupedMasked
                                   ? uint64_t(MaskedSlots(num_groups, m, n, BLOCK_M, BLOCK_N, expected_m).num_slots())
                                   : (BLOCK_M == 256 ? uint64_t(ContiguousSlots::num_slots(m, n, BLOCK_M, BLOCK_N)) : uint64_t(sched.grid_size()));
        if (slots >= kOutOfRange) return hipErrorInvalidValue;
        const int grid = capped_grid(int(slots), num_sms, device_cu_count());
        hipLaunchKernelGGL((fp8_gemm_kernel<SHAPE_N, SHAPE_K, BLOCK_M, BLOCK_N, kGemmType, int(kNumStages)>), dim3(grid),
                           dim3(fp8_launch_waves(BLOCK_M, BLOCK_N, int(kNumStages)) * kWaveSize), 0, stream, static_cast<const uint8_t*>(lhs), lhs_scales,
                           static_cast<const uint8_t*>(rhs), rhs_scales, reinterpret_cast<__bf16*>(out), m, n, k,
                           lhs_scales_stride_m, lhs_scales_stride_k, grouped_layout, lhs_scales_stride_g, int(slots), num_groups,
                           expected_m);
        return hipGetLastError();
    }

    // The contiguous layout with the tile height chosen on the device, tile row by tile row (fp8_gemm_contiguous_rows_kernel):
    // 256 x BLOCK_N tiles where a tile row holds one group, 128 x BLOCK_N where it holds two. Arguments as run_grouped.
    static hipError_t run_grouped_rows_on_device(__hip_bfloat16* out, const void* lhs, const float* lhs_scales, int lhs_scales_stride_m,
                                                 int lhs_scales_stride_k, const void* rhs, const float* rhs_scales,
                                                 const int* grouped_layout, int num_groups, int m, int n, int k, hipStream_t stream,
                                                 int num_sms = 0) {
        static_assert(kGemmType == GemmType::GroupedContiguous && BLOCK_M == 256 && kNumStages == 2);
        if (m == 0 || n == 0 || num_groups == 0) return hipSuccess;
        if (m < 0 || n < 0 || k <= 0 || num_groups < 0 || (n % 4) != 0 || (k % 128) != 0 || (m % 128) != 0) return hipErrorInvalidValue;
        if ((SHAPE_N && n != int(SHAPE_N)) || (SHAPE_K && k != int(SHAPE_K))) return hipErrorInvalidValue;
        if (kNumGroups > 1 && num_groups != int(kNumGroups)) return hipErrorInvalidValue;
        if (!out || !lhs || !lhs_scales || !rhs || !rhs_scales || !grouped_layout) return hipErrorInvalidValue;
        const uint64_t m_pad = uint64_t(ceil_div<uint32_t>(m, BLOCK_M)) * BLOCK_M, n_pad = uint64_t(ceil_div<uint32_t>(n, BLOCK_N)) * BLOCK_N;
        if (m_pad * k >= kOutOfRange || n_pad * k >= kOutOfRange || uint64_t(BLOCK_M) * n * 2 >= kOutOfRange) return hipErrorInvalidValue;
        // whole tiles (rounded up to the 8 XCDs) plus two half tiles for every other tile: at most the tiles of the 128-row tiling + 8
        const long long slots = (long long)XcdTileScheduler<>(m, n, 128, BLOCK_N).grid_size() + kNumXCD;
        if (slots >= kOutOfRange) return hipErrorInvalidValue;
        const int grid = capped_grid(int(slots), num_sms, device_cu_count());
        hipLaunchKernelGGL((fp8_gemm_contiguous_rows_kernel<SHAPE_N, SHAPE_K, BLOCK_N>), dim3(grid), dim3(8 * kWaveSize), 0, stream,
                           static_cast<const uint8_t*>(lhs), lhs_scales, static_cast<const uint8_t*>(rhs), rhs_scales,
                           reinterpret_cast<__bf16*>(out), m, n, k, lhs_scales_stride_m, lhs_scales_stride_k, grouped_layout, num_groups);
        return hipGetLastError();
    }

    // K split SPLIT_K ways over as many workgroups per tile (plain GEMM, ring tiles). `workspace` is device memory of at
    // least split_k_workspace_bytes<SPLIT_K>(m, n) bytes: kSplitKCounterBytes of arrival counters, which must be zero before
    // the first launch that uses the workspace and are zero again after every launch, then the partial sums. Launches of
    // any shapes may share a workspace one after the other; launches that share one must not overlap.
    template <int SPLIT_K>
    static size_t split_k_workspace_bytes(int m, int n) {
        const XcdTileScheduler<> sched(m, n, BLOCK_M, BLOCK_N);
        return kSplitKCounterBytes + size_t(sched.grid_size()) * SPLIT_K * BLOCK_M * BLOCK_N * 4;
    }
    template <int SPLIT_K>
    static hipError_t run_split_k(__hip_bfloat16* out, const void* lhs, const float* lhs_scales, int lhs_scales_stride_m,
                                  int lhs_scales_stride_k, const void* rhs, const float* rhs_scales, int m, int n, int k,
                                  hipStream_t stream, void* workspace, size_t workspace_bytes) {
        static_assert(kGemmType == GemmType::Normal && SPLIT_K > 1);
        if (m == 0 || n == 0) return hipSuccess;
        if (m < 0 || n < 0 || k <= 0 || (n % 4) != 0 || (k % 128) != 0) return hipErrorInvalidValue;
        if ((SHAPE_N && n != int(SHAPE_N)) || (SHAPE_K && k != int(SHAPE_K))) return hipErrorInvalidValue;
        if (!out || !lhs || !lhs_scales || !rhs || !rhs_scales || !workspace) return hipErrorInvalidValue;
        const uint64_t m_pad = uint64_t(ceil_div<uint32_t>(m, BLOCK_M)) * BLOCK_M, n_pad = uint64_t(ceil_div<uint32_t>(n, BLOCK_N)) * BLOCK_N;
        if (m_pad * k >= kOutOfRange || n_pad * k >= kOutOfRange) return hipErrorInvalidValue;
        if (uint64_t(BLOCK_M) * n * 2 >= kOutOfRange) return hipErrorInvalidValue;
        const XcdTileScheduler<> sched(m, n, BLOCK_M, BLOCK_N);
        // a counter per tile slot and wave; a workgroup per tile slot and part
        if (uint64_t(sched.grid_size()) * Fp8TileConfig<BLOCK_M, BLOCK_N>::NUM_WAVES * 4 > kSplitKCounterBytes) return hipErrorInvalidValue;
        if (workspace_bytes < split_k_workspace_bytes<SPLIT_K>(m, n)) return hipErrorInvalidValue;
        const long long grid = (long long)sched.grid_size() * SPLIT_K;
        unsigned* counters = static_cast<unsigned*>(workspace);
        float* partials = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + kSplitKCounterBytes);
        hipLaunchKernelGGL((fp8_gemm_split_k_kernel<SHAPE_N, SHAPE_K, BLOCK_M, BLOCK_N, int(kNumStages), SPLIT_K>), dim3(int(grid)),
                           dim3(fp8_launch_waves(BLOCK_M, BLOCK_N, int(kNumStages)) * kWaveSize), 0, stream, static_cast<const uint8_t*>(lhs), lhs_scales,
                           static_cast<const uint8_t*>(rhs), rhs_scales, reinterpret_cast<__bf16*>(out), m, n, k,
                           lhs_scales_stride_m, lhs_scales_stride_k, partials, counters);
        return hipGetLastError();
    }

    // Same with explicit n and k, which must equal SHAPE_N / SHAPE_K unless those are 0 (sizes known at run time).
    static hipError_t run_sized(__hip_bfloat16* out, const void* lhs, const float* lhs_scales, int lhs_scales_stride_m,
                                int lhs_scales_stride_k, const void* rhs, const float* rhs_scales, int m, int n, int k,
                                hipStream_t stream, int num_sms, uint32_t smem_size) {
        (void)smem_size;
        if (m == 0 || n == 0) return hipSuccess;
        if (m < 0 || n < 0 || k <= 0 || (n % 4) != 0 || (k % 128) != 0) return hipErrorInvalidValue;
        if ((SHAPE_N && n != int(SHAPE_N)) || (SHAPE_K && k != int(SHAPE_K))) return hipErrorInvalidValue;
        if (!out || !lhs || !lhs_scales || !rhs || !rhs_scales) return hipErrorInvalidValue;
        // 32-bit descriptor offsets: every tile row, including the overhang of the last tile, must stay below 2 GiB
        const uint64_t m_pad = uint64_t(ceil_div<uint32_t>(m, BLOCK_M)) * BLOCK_M, n_pad = uint64_t(ceil_div<uint32_t>(n, BLOCK_N)) * BLOCK_N;
        if (m_pad * k >= kOutOfRange || n_pad * k >= kOutOfRange) return hipErrorInvalidValue;
        // output stores address a tile with 32-bit byte offsets from its first element: BLOCK_M rows of n elements
        if (uint64_t(BLOCK_M) * n * 2 >= kOutOfRange) return hipErrorInvalidValue;
        using Cfg = Fp8TileConfig<BLOCK_M, BLOCK_N>;
        const XcdTileScheduler<> sched(m, n, BLOCK_M, BLOCK_N);
        const int slots = sched.grid_size();
        int grid = capped_grid(slots, num_sms, device_cu_count());
        if (fp8_walks<int(kNumStages), GemmType::Normal>(k)) {
            // persistent: one workgroup per CU (a multiple of the 8 XCDs, so a workgroup's tiles stay on one XCD), or as
            // many as the caller's cap allows
            const int cus = device_cu_count() / kNumXCD * kNumXCD;
            grid = capped_grid(slots < cus ? slots : cus, num_sms, device_cu_count());
        }
        hipLaunchKernelGGL((fp8_gemm_kernel<SHAPE_N, SHAPE_K, BLOCK_M, BLOCK_N, GemmType::Normal, int(kNumStages)>), dim3(grid),
                           dim3(fp8_launch_waves(BLOCK_M, BLOCK_N, int(kNumStages)) * kWaveSize), 0, stream, static_cast<const uint8_t*>(lhs), lhs_scales,
                           static_cast<const uint8_t*>(rhs), rhs_scales, reinterpret_cast<__bf16*>(out), m, n, k,
                           lhs_scales_stride_m, lhs_scales_stride_k, static_cast<const int*>(nullptr), 0, slots, 1, 0);
        return hipGetLastError();
    }
};

} // namespace yan
