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
// and three more that add the other ingredients of the block-scaled kernel's main loop to pattern 3, one at a time, on a
// 256 x 256 x 128 tile that never changes (so nothing but the named ingredient is added):
//   4  + the operand fragments are re-read from LDS every k-tile (24 ds_read_b128 per wave per 32 MFMAs)
//   5  + a workgroup barrier per k-tile
//   6  + the k-tile's 64 KB of copies (buffer_load ... lds) from a 64 KB region that stays in L2
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

// Patterns 4..6: the fold loop of pattern 3 fed the way the GEMM kernel is fed. `src` holds 128 KB per workgroup.
template <int MODE>
__global__ void __launch_bounds__(512) mfma_ceiling_fed_kernel(const i32x4* __restrict__ src, float* __restrict__ out, int iters) {
    __shared__ __attribute__((aligned(1024))) i32x4 lds[2][4096];      // the stage that is read, and the stage copied into
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wn = wave & 1, wm = wave >> 1;
    const i32x4* mine = src + size_t(blockIdx.x) * 8192;
    for (int i = threadIdx.x; i < 4096; i += 512) lds[0][i] = mine[i];
    __syncthreads();
    const int g = lane / 16, row = lane % 16;
    auto slot = [&](int r, int c) { return r * 8 + (c ^ (r & 7) ^ ((r >> 3) & 1)); };          // 16-byte slots, swizzled
    auto frag = [&](const i32x4* tile, int row0) {
        const i32x4 lo = tile[slot(row0 + row, 2 * g)], hi = tile[slot(row0 + row, 2 * g + 1)];
        return i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    const i32x4* ta = lds[0] + wm * 64 * 8;                 // this wave's 64 activation rows (rows 0..255 of the stage)
    const i32x4* tb = lds[0] + 2048 + wn * 128 * 8;         // its 128 weight rows (rows 256..511)
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<i32x4*>(mine + 4096), 0, 65536, 0x00020000);
    f32x4 acc[8][4] = {};
    const float scale[4] = {0.001f, 0.0015f, 0.00075f, 0.00125f};
    for (int it = 0; it < iters; ++it) {
        if constexpr (MODE >= 5) {
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, kNoWaitLgkm));
            __syncthreads();
        }
        i32x8 b[4], nf[2];
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = frag(ta, j * 16);
        nf[0] = frag(tb, 0);
        f32x4 p[4];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 34; ++t) {
            if (t < 32) {
                const int i = t / 4, j = t % 4;
                if (j == 0 && i + 1 < 8) nf[(i + 1) & 1] = frag(tb, (i + 1) * 16);
                if (MODE >= 6 && j == 1 && i < 4) {         // 8 copies per wave per k-tile over the first four rows of atoms
#pragma unroll
                    for (int c = 0; c < 2; ++c) {
                        const int q = (i * 2 + c) * 8 + wave;
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, YAN_LDS_PTR(&lds[1][0] + q * 64), 16, lane * 16, q * 1024, 0, 0);
                    }
                }
                p[t % 4] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(nf[i & 1], b[j], f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
            }
            if (t >= 2) {
                const int u = t - 2;
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[u / 4][u % 4][r] = __builtin_fmaf(p[u % 4][r], scale[u % 4], acc[u / 4][u % 4][r]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) sum += acc[i][j][r];
    out[size_t(blockIdx.x) * blockDim.x + threadIdx.x] = sum;
}

// Floating-point operations one launch performs (every CU gets one workgroup).
inline double mfma_ceiling_flops(int mode, int num_cus, int iters) {
    const double per_wave_iter = mode == 0 ? 16.0 * 2 * 32 * 32 * 16 : (mode == 1 ? 16.0 * 2 * 16 * 16 * 32 : 32.0 * 2 * 16 * 16 * 128);
    return per_wave_iter * (mode == 0 ? 4 : 8) * double(num_cus) * iters;
}

// src: num_cus * 8 * 12 * 64 * 32 bytes of operand bits (196 KB per workgroup; patterns 4..6 use the first 128 KB of each); out: num_cus * 512 floats. Returns hipSuccess or an error.
inline hipError_t launch_mfma_ceiling(int mode, const void* src, float* out, int num_cus, int iters, hipStream_t stream) {
    if (mode < 0 || mode > 6 || !src || !out || num_cus <= 0 || iters <= 0) return hipErrorInvalidValue;
    const i32x8* s = static_cast<const i32x8*>(src);
    if (mode == 0) hipLaunchKernelGGL((mfma_ceiling_kernel<0>), dim3(num_cus), dim3(256), 0, stream, s, out, iters);
    if (mode == 1) hipLaunchKernelGGL((mfma_ceiling_kernel<1>), dim3(num_cus), dim3(512), 0, stream, s, out, iters);
    if (mode == 2) hipLaunchKernelGGL((mfma_ceiling_kernel<2>), dim3(num_cus), dim3(512), 0, stream, s, out, iters);
    if (mode == 3) hipLaunchKernelGGL((mfma_ceiling_kernel<3>), dim3(num_cus), dim3(512), 0, stream, s, out, iters);
    const i32x4* f = static_cast<const i32x4*>(src);
    if (mode == 4) hipLaunchKernelGGL((mfma_ceiling_fed_kernel<4>), dim3(num_cus), dim3(512), 0, stream, f, out, iters);
    if (mode == 5) hipLaunchKernelGGL((mfma_ceiling_fed_kernel<5>), dim3(num_cus), dim3(512), 0, stream, f, out, iters);
    if (mode == 6) hipLaunchKernelGGL((mfma_ceiling_fed_kernel<6>), dim3(num_cus), dim3(512), 0, stream, f, out, iters);
    return hipGetLastError();
}

} // namespace yan
