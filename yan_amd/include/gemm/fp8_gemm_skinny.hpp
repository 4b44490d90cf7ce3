// Block-scaled FP8 GEMM for a handful of activation rows (the launcher sends m <= 16 here): bound by streaming the
// weights out of HBM once, not by the matrix core. Above that the tiled kernel with its ring of LDS stages is as
// fast or faster (it reads the activations once per 16..128 weight rows through LDS instead of once per 16 from L2).
//
// Same contract as fp8_gemm.hpp (operands of yan/jit_kernels/gemm.py:23-30, scale granularity of
// yan/include/gemm/fp8_gemm.cuh:48-61); a different kernel, because the tiled one keeps one k-tile per CU in
// flight and a 64-row problem has too few tiles to fill 256 CUs:
//   * one workgroup per 16 weight rows (N/16 workgroups: 256 for N = 4096), every CU pulling its own slice of B;
//   * no LDS staging and no barriers in the main loop: wave w of a workgroup owns K blocks w, w+W, w+2W, ... and
//     streams their operand fragments straight into registers, DEPTH blocks ahead, so each wave keeps
//     DEPTH x (2 + 2*TM) 16-byte loads per lane in flight and the compiler's per-register waits do the rest;
//   * per K block: one 16x16x128 MFMA per 16 activation rows from a zero accumulator, folded in with
//     acc += p * (sA * sB) exactly as the tiled kernel does;
//   * the W partial sums of a workgroup meet once, through 16 KB of LDS, and leave as bf16.
// The activations are re-read from L2 by every workgroup (m*K bytes each); for m = 64 that is 117 MB of L2 traffic
// next to 29 MB of HBM traffic, which the L2s sustain.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>

#include "utils.hpp"
#include "mfma_utils.hpp"
#include "tile_io.hpp"

namespace yan {

// TM: 16-row activation atoms covered (m <= 16*TM). NUM_WAVES: waves sharing the K blocks of one workgroup.
template <int SHAPE_N, int SHAPE_K, int TM, int NUM_WAVES>
__global__ void __launch_bounds__(NUM_WAVES * kWaveSize)
fp8_gemm_skinny_kernel(const uint8_t* __restrict__ lhs, const float* __restrict__ lhs_scales,
                       const uint8_t* __restrict__ rhs, const float* __restrict__ rhs_scales,
                       __bf16* __restrict__ out, int m, int n_rt, int k_rt, int sa_stride_m, int sa_stride_k) {
    using Atom = MfmaFP8_16x16x128;
    constexpr int DEPTH = TM <= 2 ? 6 : (TM <= 4 ? 4 : 2);          // K blocks in flight per wave
    static_assert(NUM_WAVES >= TM, "the final reduction gives one activation atom to each of the first TM waves");
    const int N = SHAPE_N ? SHAPE_N : n_rt, K = SHAPE_K ? SHAPE_K : k_rt;
    const int NUM_K_BLOCKS = K / 128, NUM_N_BLOCKS = ceil_div(N, 128);

    __shared__ __attribute__((aligned(16))) float partial[NUM_WAVES][TM][kWaveSize][4];

    const int n0 = blockIdx.x * 16;
    const int lane = get_lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const int g = lane / 16, col = lane % 16;

    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(lhs, uint32_t(m) * K);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(rhs, uint32_t(N) * K);
    const uint32_t sa_bytes = (uint32_t(m - 1) * sa_stride_m + uint32_t(NUM_K_BLOCKS - 1) * sa_stride_k + 1) * 4;
    const __amdgpu_buffer_rsrc_t rsrc_sa = make_rsrc(lhs_scales, sa_bytes);
    // Lane (col, g) holds bytes [32g, 32g+32) of K block kb of row `col` of its atom, for both operands; rows past
    // the end of either matrix start beyond num_records and read as zero.
    const uint32_t voff_b = uint32_t(n0 + col) * K + 32 * g;
    const uint32_t voff_a = uint32_t(col) * K + 32 * g;
    const uint32_t voff_sa = uint32_t(col) * sa_stride_m * 4;
    const float* sb_row = rhs_scales + size_t(min(n0 / 128, NUM_N_BLOCKS - 1)) * NUM_K_BLOCKS;

    // Every workgroup reads all of the activations. Left alone they would all want the same few cache lines at the
    // same moment and queue on the L2 channels that hold them; starting each workgroup at a different K block (and
    // wrapping around) spreads the requests over the whole activation matrix.
    const int rot = (blockIdx.x * 7) % NUM_K_BLOCKS;
    auto rotated = [&](int kb) { const int r = kb + rot; return r >= NUM_K_BLOCKS ? r - NUM_K_BLOCKS : r; };

    struct Stage {
        i32x4 b[2];
        i32x4 a[TM][2];
        float sa[TM];
        float sb;
    };
    Stage st[DEPTH];
    auto load = [&](Stage& s, int seq) {
        const bool valid = seq < NUM_K_BLOCKS;          // past the end: operands read as zero, scales as some block's
        const uint32_t vb = valid ? voff_b : kOutOfRange, va = valid ? voff_a : kOutOfRange;
        const int kb = rotated(min(seq, NUM_K_BLOCKS - 1)), kbc = kb;
        s.b[0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vb, kb * kRowBytes, 0);
        s.b[1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vb, kb * kRowBytes + 16, 0);
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            s.a[j][0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, va, kb * kRowBytes + j * 16 * K, 0);
            s.a[j][1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, va, kb * kRowBytes + j * 16 * K + 16, 0);
            s.sa[j] = buffer_load_f32(rsrc_sa, voff_sa, (kbc * sa_stride_k + j * 16 * sa_stride_m) * 4);
        }
        s.sb = sb_row[kbc];
    };

    f32x4 acc[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
    for (int s = 0; s < DEPTH; ++s) load(st[s], wave + s * NUM_WAVES);
    for (int kb = wave; kb < NUM_K_BLOCKS; kb += DEPTH * NUM_WAVES) {
#pragma unroll
        for (int s = 0; s < DEPTH; ++s) {
            const Stage& c = st[s];
            const i32x8 bf = {c.b[0][0], c.b[0][1], c.b[0][2], c.b[0][3], c.b[1][0], c.b[1][1], c.b[1][2], c.b[1][3]};
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                const i32x8 af = {c.a[j][0][0], c.a[j][0][1], c.a[j][0][2], c.a[j][0][3],
                                  c.a[j][1][0], c.a[j][1][1], c.a[j][1][2], c.a[j][1][3]};
                const f32x4 p = Atom::mma(bf, af, f32x4{0.f, 0.f, 0.f, 0.f});
                const float scale = c.sa[j] * c.sb;
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[j][r] = __builtin_fmaf(p[r], scale, acc[j][r]);
            }
            load(st[s], kb + (s + DEPTH) * NUM_WAVES);
        }
    }

    // Meet the other waves' partial sums: wave j < TM finishes activation atom j.
#pragma unroll
    for (int j = 0; j < TM; ++j) *reinterpret_cast<f32x4*>(partial[wave][j][lane]) = acc[j];
    __syncthreads();
    if (wave < TM) {
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < NUM_WAVES; ++w) sum += *reinterpret_cast<const f32x4*>(partial[w][wave][lane]);
        // the 4 registers are n = n0 + 4g + {0..3} of row m = 16*wave + col
        const int mm = wave * 16 + col, nn = n0 + 4 * g;
        if (mm < m && nn < N) *reinterpret_cast<bf16x4*>(out + size_t(mm) * N + nn) = pack4(sum, __bf16{});
    }
}

// Launcher for m <= 16*TM. Returns hipErrorInvalidValue for sizes outside the kernel's reach.
template <int SHAPE_N, int SHAPE_K, int TM, int NUM_WAVES>
inline hipError_t launch_fp8_skinny(__hip_bfloat16* out, const void* lhs, const float* lhs_scales, int lhs_scales_stride_m,
                                    int lhs_scales_stride_k, const void* rhs, const float* rhs_scales, int m, int n, int k,
                                    hipStream_t stream) {
    if (m == 0 || n == 0) return hipSuccess;
    if (m < 0 || m > 16 * TM || n < 0 || k <= 0 || (n % 4) != 0 || (k % 128) != 0) return hipErrorInvalidValue;
    if ((SHAPE_N && n != SHAPE_N) || (SHAPE_K && k != SHAPE_K)) return hipErrorInvalidValue;
    if (!out || !lhs || !lhs_scales || !rhs || !rhs_scales) return hipErrorInvalidValue;
    if (uint64_t(16 * TM) * k >= kOutOfRange || (uint64_t(n) + 16) * k >= kOutOfRange) return hipErrorInvalidValue;
    hipLaunchKernelGGL((fp8_gemm_skinny_kernel<SHAPE_N, SHAPE_K, TM, NUM_WAVES>), dim3(ceil_div(n, 16)),
                       dim3(NUM_WAVES * kWaveSize), 0, stream, static_cast<const uint8_t*>(lhs), lhs_scales,
                       static_cast<const uint8_t*>(rhs), rhs_scales, reinterpret_cast<__bf16*>(out), m, n, k,
                       lhs_scales_stride_m, lhs_scales_stride_k);
    return hipGetLastError();
}

} // namespace yan
