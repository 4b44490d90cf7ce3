// C = alpha * A . B^T + beta * C in fp32 on gfx950, operands stored the way the reference's fp32 GEMM takes them.
//
// Entry point `gemm_nt(m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC, stream)` keeps the name, argument order and
// memory convention of the reference's launcher (yan/include/gemm/simple_gemm.cuh:194-247): A is m x k with M
// contiguous (element (i, kk) at A[i + kk * ldA]), B is n x k with N contiguous (B[j + kk * ldB]), C is m x n
// row-major (C[i * ldC + j]), work is enqueued on `stream`. The reference kernel (simple_gemm.cuh:16-192) is a
// 128 x 64 x 16 cp.async pipeline of scalar FMAs; here:
//   * macro tile BLOCK_M x BLOCK_N, 16 to 128 k-rows per LDS stage, 4 waves in a 2 x 2 arrangement, one per SIMD, each with a
//     (BLOCK_M / 2) x (BLOCK_N / 2) slab of 32x32x2 fp32 MFMAs (up to 128 x 128: 256 accumulator registers);
//   * a k-row of a tile is contiguous in memory, so one buffer_load ... lds instruction moves 1 KB of it (or two
//     k-rows of a 128-wide tile) to where the fragments are read from; a ring of LDS stages keeps
//     NUM_STAGES - 1 k-tiles in flight;
//   * a lane reads VM = BLOCK_M / 64 consecutive floats of one k-row as the row operands of VM MFMAs (and VN
//     floats for the columns), which makes MFMA t of a slab cover the rows VM * i + t: a lane's VN column
//     accumulators are VN consecutive n of one m, one 16-byte access in C;
//   * tiles below 128 rows (64 x 64, 32 x 64, 32 x 32) are for problems with too few outputs to give every CU a
//     large tile: there the four waves split K instead of the tile (each takes a quarter of every 64-deep k-tile
//     over the whole tile) and their partial sums are added through LDS in a fixed order at the end, so results do
//     not depend on timing;
//   * rows past m / n are not written, k rows past the end read as zero: any m, n, k with m, n, ldA, ldB, ldC
//     multiples of 4 and 16-byte aligned bases.
// beta == 0 does not read C (the BLAS convention).
#pragma once

#include <hip/hip_runtime.h>

#include "utils.hpp"
#include "mfma_utils.hpp"
#include "scheduler.hpp"
#include "tile_io.hpp"

namespace yan {

template <int BLOCK_M, int BLOCK_N>
struct FloatTileConfig {
    static constexpr int NUM_WAVES = 4;
    static constexpr int K_SPLIT = BLOCK_M < 128 ? 4 : 1;                    // waves that share one tile along K
    static constexpr int WAVES_M = K_SPLIT == 4 ? 1 : 2, WAVES_N = WAVES_M;
    // k-rows per LDS stage: 16 to 32 KB of operands, and a barrier between k-tiles once per 2000-8000 MFMA cycles
    static constexpr int BLOCK_K = K_SPLIT == 4 ? 64 : (BLOCK_M + BLOCK_N >= 256 ? 16 : 32);
    static constexpr int KP_PER_WAVE = BLOCK_K / 2 / K_SPLIT;                // k-pairs (one MFMA deep) per wave per k-tile
    static constexpr int WTM = BLOCK_M / WAVES_M, WTN = BLOCK_N / WAVES_N;
    static constexpr int VM = WTM / 32, VN = WTN / 32;                       // floats per lane per operand read
    static_assert((VM == 1 || VM == 2 || VM == 4) && (VN == 1 || VN == 2 || VN == 4), "slabs of 32, 64 or 128 per side");
    static constexpr int A_BYTES = BLOCK_K * BLOCK_M * 4, B_BYTES = BLOCK_K * BLOCK_N * 4;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int A_COPIES = A_BYTES / 1024, B_COPIES = B_BYTES / 1024;     // wave instructions per stage
    static_assert(A_COPIES % NUM_WAVES == 0 && B_COPIES % NUM_WAVES == 0);
    static constexpr int OPS = (A_COPIES + B_COPIES) / NUM_WAVES;                // per wave per k-tile
    static_assert(OPS <= KP_PER_WAVE, "one copy per k-pair");
    // The 128 x 128 and 128 x 64 tiles and the two smallest ones keep their ring within 72 KB so that two workgroups
    // fit a CU and cover each other's barriers (measured: 2-10 % and 5-25 % faster than one workgroup with a
    // deeper ring).
    static constexpr int RING_BUDGET = (BLOCK_M == 32 || (BLOCK_M == 128 && BLOCK_N <= 128)) ? 72 * 1024 : 128 * 1024;
    static constexpr int MAX_STAGES = RING_BUDGET / STAGE_BYTES < 3 ? 3 : (RING_BUDGET / STAGE_BYTES < 8 ? RING_BUDGET / STAGE_BYTES : 8);
    static_assert(K_SPLIT == 1 || 3 * VM * VN * 16 * 256 <= 3 * STAGE_BYTES, "partial sums of three waves fit the ring");
};

template <int N> struct FloatVec;
template <> struct FloatVec<1> { using type = float; };
template <> struct FloatVec<2> { typedef float type __attribute__((ext_vector_type(2))); };
template <> struct FloatVec<4> { using type = f32x4; };

template <int N>
__device__ __forceinline__ float vec_at(const typename FloatVec<N>::type& v, int i) {
    if constexpr (N == 1) return v; else return v[i];
}

// The kernel keeps the reference kernel's name (simple_gemm.cuh:22) so that profiler filters written for it
// (tests/test_simple.py:35 looks for 'gemm_cute') keep finding it.
template <int BLOCK_M, int BLOCK_N, int STAGES>
__global__ void __launch_bounds__(4 * kWaveSize)
gemm_cute(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C,
          int m, int n, int k, int ldA, int ldB, int ldC, float alpha, float beta) {
    using Cfg = FloatTileConfig<BLOCK_M, BLOCK_N>;
    constexpr int VM = Cfg::VM, VN = Cfg::VN, BLOCK_K = Cfg::BLOCK_K, OPS = Cfg::OPS;
    static_assert(STAGES >= 3 && STAGES <= Cfg::MAX_STAGES && (STAGES - 2) * OPS <= 63);
    using VecM = typename FloatVec<VM>::type;
    using VecN = typename FloatVec<VN>::type;

    const XcdTileScheduler<> sched(m, n, BLOCK_M, BLOCK_N);
    const TileCoord tile = sched.tile_of(blockIdx.x);
    if (!tile.valid) return;
    const int m0 = tile.m_idx * BLOCK_M, n0 = tile.n_idx * BLOCK_N;

    const int lane = get_lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const int wm = Cfg::K_SPLIT == 4 ? 0 : wave / Cfg::WAVES_N, wn = Cfg::K_SPLIT == 4 ? 0 : wave % Cfg::WAVES_N;

    // Descriptors end with the last element of the last k-row, so every k-row past k reads as zero.
    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(A, k > 0 ? (uint32_t(k - 1) * uint32_t(ldA) + uint32_t(m)) * 4u : 0u);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(B, k > 0 ? (uint32_t(k - 1) * uint32_t(ldB) + uint32_t(n)) * 4u : 0u);
    // One copy instruction moves 1 KB of a stage: 1024 / (4 * BLOCK) consecutive k-rows of BLOCK floats each.
    constexpr int A_LANES = BLOCK_M / 4, B_LANES = BLOCK_N / 4;                 // lanes per k-row
    constexpr int A_ROWS = kWaveSize / A_LANES, B_ROWS = kWaveSize / B_LANES;   // k-rows per instruction
    const uint32_t voff_a = (uint32_t(lane / A_LANES) * uint32_t(ldA) + uint32_t(m0 + (lane % A_LANES) * 4)) * 4u;
    const uint32_t voff_b = (uint32_t(lane / B_LANES) * uint32_t(ldB) + uint32_t(n0 + (lane % B_LANES) * 4)) * 4u;
    // Copy number `d` of this wave (A instructions first, then B) of k-tile `kt` into the stage at `stage`.
    auto copy_op = [&](int d, int kt, uint8_t* stage) {
        const int q = d * Cfg::NUM_WAVES + wave;
        if (d < Cfg::A_COPIES / Cfg::NUM_WAVES) {
            const uint32_t k_row = uint32_t(kt * BLOCK_K + q * A_ROWS);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, YAN_LDS_PTR(stage + q * 1024), kChunk, voff_a, k_row * uint32_t(ldA) * 4u, 0, 0);
        } else {
            const int qb = q - Cfg::A_COPIES;
            const uint32_t k_row = uint32_t(kt * BLOCK_K + qb * B_ROWS);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, YAN_LDS_PTR(stage + Cfg::A_BYTES + qb * 1024), kChunk, voff_b, k_row * uint32_t(ldB) * 4u, 0, 0);
        }
    };

    f32x16 acc[VM][VN];
#pragma unroll
    for (int t = 0; t < VM; ++t)
#pragma unroll
        for (int u = 0; u < VN; ++u)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][u][r] = 0.f;

    // Lane (h, i) = (lane / 32, lane % 32) supplies k-row 2 * kp + h of k-pair kp: VM floats from column VM * i of
    // its slab of the A part, VN floats from column VN * i of its slab of the B part.
    const int h = lane / 32, i = lane % 32;
    // With K split over the waves, wave w owns k-pairs KP_PER_WAVE * w .. of every k-tile.
    const int first_kp = Cfg::K_SPLIT == 4 ? wave * Cfg::KP_PER_WAVE : 0;
    const int frag_a = ((2 * first_kp + h) * BLOCK_M + wm * Cfg::WTM + VM * i) * 4;
    const int frag_b = Cfg::A_BYTES + ((2 * first_kp + h) * BLOCK_N + wn * Cfg::WTN + VN * i) * 4;

    __shared__ __attribute__((aligned(1024))) uint8_t ring[STAGES * Cfg::STAGE_BYTES];
    const int num_k_tiles = ceil_div(k, BLOCK_K);
#pragma unroll
    for (int t = 0; t < STAGES - 1; ++t)
#pragma unroll
        for (int d = 0; d < OPS; ++d) copy_op(d, t, ring + t * Cfg::STAGE_BYTES);

    // Every wave issues OPS copies per k-tile in the same order, so "k-tile kt has landed" is "at most
    // (STAGES - 2) * OPS of my copies are outstanding"; the copies of k-tile kt + STAGES - 1 go to the stage consumed
    // in iteration kt - 1, which every wave has left once it is past the barrier.
    int st = 0;
    for (int kt = 0; kt < num_k_tiles; ++kt) {
        __builtin_amdgcn_s_waitcnt(waitcnt_imm((STAGES - 2) * OPS, kNoWaitLgkm));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const uint8_t* cur = ring + st * Cfg::STAGE_BYTES;
        uint8_t* nxt = ring + (st == 0 ? STAGES - 1 : st - 1) * Cfg::STAGE_BYTES;
        VecM fa[2];
        VecN fb[2];
        fa[0] = *reinterpret_cast<const VecM*>(cur + frag_a);
        fb[0] = *reinterpret_cast<const VecN*>(cur + frag_b);
#pragma unroll
        for (int kp = 0; kp < Cfg::KP_PER_WAVE; ++kp) {
            if (kp + 1 < Cfg::KP_PER_WAVE) {
                fa[(kp + 1) & 1] = *reinterpret_cast<const VecM*>(cur + frag_a + (kp + 1) * 2 * BLOCK_M * 4);
                fb[(kp + 1) & 1] = *reinterpret_cast<const VecN*>(cur + frag_b + (kp + 1) * 2 * BLOCK_N * 4);
            }
            // the next k-tile's copies, one per k-pair from the start of the tile
            if (kp < OPS) copy_op(kp, kt + STAGES - 1, nxt);
#pragma unroll
            for (int t = 0; t < VM; ++t)
#pragma unroll
                for (int u = 0; u < VN; ++u)
                    acc[t][u] = __builtin_amdgcn_mfma_f32_32x32x2f32(vec_at<VM>(fa[kp & 1], t), vec_at<VN>(fb[kp & 1], u), acc[t][u], 0, 0, 0);
        }
        st = st + 1 == STAGES ? 0 : st + 1;
    }

    if constexpr (Cfg::K_SPLIT == 4) {
        // Partial sums of waves 1..3 go through LDS (register-major, lane-minor: no bank conflicts) and wave 0 adds
        // them in the order 1, 2, 3. The ring is free once nobody reads it and no copy is still on its way into it.
        constexpr int REGS = VM * VN * 16;
        wait_for_copies();
        __syncthreads();
        float* partial = reinterpret_cast<float*>(ring);
        if (wave != 0) {
#pragma unroll
            for (int t = 0; t < VM; ++t)
#pragma unroll
                for (int u = 0; u < VN; ++u)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        partial[((wave - 1) * REGS + (t * VN + u) * 16 + r) * kWaveSize + lane] = acc[t][u][r];
        }
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int w = 0; w < 3; ++w)
#pragma unroll
            for (int t = 0; t < VM; ++t)
#pragma unroll
                for (int u = 0; u < VN; ++u)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        acc[t][u][r] += partial[(w * REGS + (t * VN + u) * 16 + r) * kWaveSize + lane];
    }

    // Epilogue: register r of an atom is MFMA row 8 * (r / 4) + 4 * h + r % 4 of MFMA column i; MFMA (t, u) holds
    // slab row VM * mfma_row + t and slab column VN * mfma_col + u.
    const int n_lane = n0 + wn * Cfg::WTN + VN * i;
    if (n_lane >= n) return;                                   // n % 4 == 0 and VN | 4: a lane's VN columns exist together
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int mfma_row = 8 * (r / 4) + 4 * h + r % 4;
#pragma unroll
        for (int t = 0; t < VM; ++t) {
            const int mm = m0 + wm * Cfg::WTM + VM * mfma_row + t;
            if (mm >= m) continue;
            VecN* dst = reinterpret_cast<VecN*>(C + size_t(mm) * ldC + n_lane);
            VecN v;
            if constexpr (VN == 1) v = alpha * acc[t][0][r];
            else {
#pragma unroll
                for (int u = 0; u < VN; ++u) v[u] = alpha * acc[t][u][r];
            }
            if (beta != 0.f) v += beta * *dst;
            *dst = v;
        }
    }
}

// Arguments the fp32 launcher checks before touching the GPU.
inline hipError_t check_float_args(int m, int n, int k, const void* a, int ldA, const void* b, int ldB, const void* c, int ldC,
                                   int block_m, int block_n) {
    if (m < 0 || n < 0 || k < 0 || (m % 4) != 0 || (n % 4) != 0) return hipErrorInvalidValue;
    if (ldA < m || ldB < n || ldC < n || (ldA % 4) != 0 || (ldB % 4) != 0 || (ldC % 4) != 0) return hipErrorInvalidValue;
    if (!c || (k > 0 && (!a || !b))) return hipErrorInvalidValue;          // with k == 0 the operands are never read
    if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c)) & 15) return hipErrorInvalidValue;
    // 32-bit descriptor offsets: the last k-row the ring prefetches (up to 8 k-tiles of at most 128 rows past the end), tile overhang
    // included, must stay below 2 GiB
    const uint64_t k_pad = uint64_t(k) + 8 * 128;
    if ((k_pad * ldA + block_m) * 4 >= kOutOfRange || (k_pad * ldB + block_n) * 4 >= kOutOfRange) return hipErrorInvalidValue;
    return hipSuccess;
}

template <int BLOCK_M, int BLOCK_N, int STAGES = FloatTileConfig<BLOCK_M, BLOCK_N>::MAX_STAGES>
inline hipError_t launch_float_nt(int m, int n, int k, float alpha, const float* A, int ldA, const float* B, int ldB,
                                  float beta, float* C, int ldC, hipStream_t stream) {
    if (m == 0 || n == 0) return hipSuccess;
    if (hipError_t e = check_float_args(m, n, k, A, ldA, B, ldB, C, ldC, BLOCK_M, BLOCK_N); e != hipSuccess) return e;
    const XcdTileScheduler<> sched(m, n, BLOCK_M, BLOCK_N);
    hipLaunchKernelGGL((gemm_cute<BLOCK_M, BLOCK_N, STAGES>), dim3(sched.grid_size()), dim3(4 * kWaveSize), 0, stream,
                       A, B, C, m, n, k, ldA, ldB, ldC, alpha, beta);
    return hipGetLastError();
}

// Tile for a problem when the caller names none: the one whose count of rounds of workgroups over `num_cus` CUs,
// times its area, times a measured cost per area, is smallest (the matrix cores run at nearly the same rate for all
// of them; larger tiles move fewer operand bytes per flop, and the K-split tiles pay for their reduction). Ties go
// to the earlier, larger tile.
struct FloatTile { int block_m, block_n; double per_area; };
constexpr FloatTile kFloatTiles[] = {{256, 256, 1.00}, {128, 256, 1.015}, {128, 128, 1.03}, {128, 64, 1.04},
                                     {64, 64, 1.13}, {32, 64, 1.13}, {32, 32, 1.25}};
inline FloatTile pick_float_tile(int m, int n, int num_cus) {
    FloatTile best = kFloatTiles[0];
    double best_cost = -1;
    for (const FloatTile& t : kFloatTiles) {
        const long long tiles = static_cast<long long>(ceil_div(m, t.block_m)) * ceil_div(n, t.block_n);
        const double cost = double(ceil_div<long long>(tiles, num_cus)) * t.block_m * t.block_n * t.per_area;
        if (best_cost < 0 || cost < best_cost) { best = t; best_cost = cost; }
    }
    return best;
}

} // namespace yan

template <int BLOCK_M, int BLOCK_N>
inline hipError_t gemm_nt(int m, int n, int k, float alpha, float const* A, int ldA, float const* B, int ldB,
                          float beta, float* C, int ldC, hipStream_t stream = 0) {
    return yan::launch_float_nt<BLOCK_M, BLOCK_N>(m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC, stream);
}

// The reference's signature, with no tile named (yan/jit_kernels/simple_gemm.py:8-16 calls it this way); `num_cus`
// is the number of compute units to plan for, the device's own when 0.
inline hipError_t gemm_nt(int m, int n, int k, float alpha, float const* A, int ldA, float const* B, int ldB,
                          float beta, float* C, int ldC, hipStream_t stream = 0, int num_cus = 0) {
    if (num_cus <= 0) {
        int device = 0;
        if (hipGetDevice(&device) != hipSuccess ||
            hipDeviceGetAttribute(&num_cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || num_cus <= 0)
            num_cus = 256;
    }
    const yan::FloatTile t = yan::pick_float_tile(m, n, num_cus);
#define YAN_FLOAT_CASE(BM, BN) if (t.block_m == BM && t.block_n == BN) return gemm_nt<BM, BN>(m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC, stream);
    YAN_FLOAT_CASE(256, 256) YAN_FLOAT_CASE(128, 256) YAN_FLOAT_CASE(128, 128) YAN_FLOAT_CASE(128, 64)
    YAN_FLOAT_CASE(64, 64) YAN_FLOAT_CASE(32, 64) YAN_FLOAT_CASE(32, 32)
#undef YAN_FLOAT_CASE
    return hipErrorInvalidValue;
}
