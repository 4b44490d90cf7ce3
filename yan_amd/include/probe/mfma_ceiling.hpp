// Register-resident MFMA loops: what the matrix cores of the whole chip sustain when nothing is fetched at all.
//
// The GEMM kernels in ../gemm are judged against the vendor's peak rates, which assume the top shader clock. Under
// a matrix-core load with realistic (non-constant) operand bits the chip runs into its power limit and lowers the
// clock, so the rate a kernel could reach at best is lower than the peak and depends on the data. These loops
// measure that ceiling on the machine at hand: every wave keeps its operand fragments in registers (loaded once from
// `src`, so their bit patterns are the caller's) and issues the same MFMA pattern as a GEMM main loop, with the same
// register blocking, for `iters` rounds. Four patterns:
//   0  bf16 32x32x16, 4 waves per CU, 4 x 4 atoms (the dense kernel's slab)
//   1  bf16 16x16x32, 8 waves per CU, 4 x 4 atoms
//   2  e4m3 16x16x128 accumulating in place, 8 waves per CU, 8 x 4 atoms
//   3  e4m3 16x16x128 from a zero accumulator + fp32 fold per atom (the block-scaled kernel's inner step)
#pragma once

#include <hip/hip_runtime.h>

#include "../gemm/utils.hpp"

namespace yan {

template <int MODE>
__global__ void __launch_bounds__(MODE == 0 ? 256 : 512) mfma_ceiling_kernel(const i32x8* __restrict__ src, float* __restrict__ out, int iters) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const i32x8* mine = src + (size_t(blockIdx.x) * 8 + wave) * 12 * 64 + lane;     // 12 fragments of 32 bytes per lane
    float sum = 0.f;
    if constexpr (MODE == 0) {
        bf16x8 a[4], b[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a[i] = reinterpret_cast<const bf16x8*>(mine + i * 64)[0];
            b[i] = reinterpret_cast<const bf16x8*>(mine + (4 + i) * 64)[0];
        }
        f32x16 acc[4][4] = {};
        for (int it = 0; it < iters; ++it)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) sum += acc[i][j][r];
    } else if constexpr (MODE == 1) {
        bf16x8 a[4], b[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a[i] = reinterpret_cast<const bf16x8*>(mine + i * 64)[0];
            b[i] = reinterpret_cast<const bf16x8*>(mine + (4 + i) * 64)[0];
        }
        f32x4 acc[4][4] = {};
        for (int it = 0; it < iters; ++it)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) sum += acc[i][j][r];
    } else {
        i32x8 a[8], b[4];
#pragma unroll
        for (int i = 0; i < 8; ++i) a[i] = mine[i * 64];
#pragma unroll
        for (int i = 0; i < 4; ++i) b[i] = mine[(8 + i) * 64];
        f32x4 acc[8][4] = {};
        const float scale[4] = {0.001f, 0.0015f, 0.00075f, 0.00125f};
        for (int it = 0; it < iters; ++it) {
            if constexpr (MODE == 2) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i], b[j], acc[i][j], 0, 0, 0, 0, 0, 0);
            } else {
                f32x4 p[4];
#pragma unroll
                for (int t = 0; t < 34; ++t) {
                    if (t < 32) p[t % 4] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[t / 4], b[t % 4], f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                    if (t >= 2) {
                        const int u = t - 2;
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[u / 4][u % 4][r] = __builtin_fmaf(p[u % 4][r], scale[u % 4], acc[u / 4][u % 4][r]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) sum += acc[i][j][r];
    }
    out[size_t(blockIdx.x) * blockDim.x + threadIdx.x] = sum;
}

// Floating-point operations one launch performs (every CU gets one workgroup).
inline double mfma_ceiling_flops(int mode, int num_cus, int iters) {
    const double per_wave_iter = mode == 0 ? 16.0 * 2 * 32 * 32 * 16 : (mode == 1 ? 16.0 * 2 * 16 * 16 * 32 : 32.0 * 2 * 16 * 16 * 128);
    return per_wave_iter * (mode == 0 ? 4 : 8) * double(num_cus) * iters;
}

// src: num_cus * 8 * 12 * 64 * 32 bytes of operand bits; out: num_cus * 512 floats. Returns hipSuccess or an error.
inline hipError_t launch_mfma_ceiling(int mode, const void* src, float* out, int num_cus, int iters, hipStream_t stream) {
    if (mode < 0 || mode > 3 || !src || !out || num_cus <= 0 || iters <= 0) return hipErrorInvalidValue;
    const i32x8* s = static_cast<const i32x8*>(src);
    if (mode == 0) hipLaunchKernelGGL((mfma_ceiling_kernel<0>), dim3(num_cus), dim3(256), 0, stream, s, out, iters);
    if (mode == 1) hipLaunchKernelGGL((mfma_ceiling_kernel<1>), dim3(num_cus), dim3(512), 0, stream, s, out, iters);
    if (mode == 2) hipLaunchKernelGGL((mfma_ceiling_kernel<2>), dim3(num_cus), dim3(512), 0, stream, s, out, iters);
    if (mode == 3) hipLaunchKernelGGL((mfma_ceiling_kernel<3>), dim3(num_cus), dim3(512), 0, stream, s, out, iters);
    return hipGetLastError();
}

} // namespace yan
