// Quantisers that feed the block-scaled FP8 GEMM: fp32 / bf16 -> e4m3 codes + fp32 scales, in one pass over HBM.
//
//   per-token:  one scale per row and 128 consecutive K   (activations; lhs_scales of the GEMM)
//   per-block:  one scale per 128 x 128 block              (weights; rhs_scales of the GEMM)
//   amax = max |x| over the group, clamped from below at 1e-4;  q = e4m3(x * (448 / amax));  scale = amax / 448
//
// This is the step in front of the GEMM entry whose operand names the reference fixes
// (yan/jit_kernels/gemm.py:23-30: lhs, lhs_scales, rhs, rhs_scales); the reference itself has no quantiser. The
// arithmetic is the recipe callers of this convention type in torch, `(x.float() * (448 / amax)).to(float8_e4m3fn)`
// and `amax / 448`, with both quotients correctly rounded: fp32 IEEE divisions, one fp32 multiply, round-to-nearest-
// even conversion. (torch itself evaluates `448.0 / amax` as reciprocal(amax) * 448, an ulp away for some amax.)
//
// Both kernels are bound by HBM traffic: (2 or 4) bytes read + 1 byte written per element, plus 4 bytes per
// group. Sixteen lanes own one 128-element group at a time, 8 elements per lane, so a wave reads 1 KB (bf16) or
// 2 KB (fp32) of consecutive addresses per step and writes 512 B.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>

#include "utils.hpp"

namespace yan {

constexpr float kFp8Max = 448.0f;

// Eight consecutive source elements as fp32.
struct F32x8 { float v[8]; };

__device__ __forceinline__ F32x8 load8(const float* p) {
    const f32x4 lo = *reinterpret_cast<const f32x4*>(p), hi = *reinterpret_cast<const f32x4*>(p + 4);
    return {{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]}};
}

__device__ __forceinline__ F32x8 load8(const __bf16* p) {
    const bf16x8 x = *reinterpret_cast<const bf16x8*>(p);
    F32x8 r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r.v[i] = float(x[i]);
    return r;
}

__device__ __forceinline__ F32x8 load8(const __hip_bfloat16* p) { return load8(reinterpret_cast<const __bf16*>(p)); }

__device__ __forceinline__ float abs_max8(const F32x8& x) {
    float a = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) a = fmaxf(a, fabsf(x.v[i]));
    return a;
}

// Eight e4m3 codes (OCP on gfx950, round to nearest even) of x * factor, packed little-endian in two dwords.
__device__ __forceinline__ uint2 quantise8(const F32x8& x, float factor) {
    int lo = 0, hi = 0;
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(x.v[0] * factor, x.v[1] * factor, lo, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(x.v[2] * factor, x.v[3] * factor, lo, true);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(x.v[4] * factor, x.v[5] * factor, hi, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(x.v[6] * factor, x.v[7] * factor, hi, true);
    return make_uint2(uint32_t(lo), uint32_t(hi));
}

// Maximum over the 16 lanes that share a group (lanes 16g .. 16g+15 of the wave).
__device__ __forceinline__ float max_over_16_lanes(float a) {
#pragma unroll
    for (int d = 8; d >= 1; d >>= 1) a = fmaxf(a, __shfl_xor(a, d, 16));
    return a;
}

// x [m, k] row-major with k % 128 == 0, seen as m*k/128 consecutive groups. Scale of (row, kb) goes to
// scales[row * stride_m + kb * stride_k]. UNROLL groups per 16 lanes are in flight at once.
template <typename T, int UNROLL>
__global__ void __launch_bounds__(256)
per_token_cast_kernel(const T* __restrict__ x, uint8_t* __restrict__ q, float* __restrict__ scales,
                      long long num_groups, int k_blocks, long long stride_m, long long stride_k) {
    const long long first = (static_cast<long long>(blockIdx.x) * UNROLL * 256 + threadIdx.x) >> 4;
    const int part = threadIdx.x & 15;
    F32x8 v[UNROLL];
    bool live[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const long long group = first + u * 16;             // 256 threads = 16 groups per step
        live[u] = group < num_groups;
        if (live[u]) v[u] = load8(x + group * 128 + part * 8);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const long long group = first + u * 16;
        float amax = live[u] ? abs_max8(v[u]) : 0.f;
        amax = fmaxf(max_over_16_lanes(amax), 1e-4f);
        if (!live[u]) continue;
        *reinterpret_cast<uint2*>(q + group * 128 + part * 8) = quantise8(v[u], kFp8Max / amax);
        if (part == 0) {
            const long long row = group / k_blocks, kb = group - row * k_blocks;
            scales[row * stride_m + kb * stride_k] = amax / kFp8Max;
        }
    }
}

// w [n, k] row-major with k % 128 == 0: one workgroup per 128 x 128 block; rows past n count as zeros and are not
// written. scales [ceil(n/128), k/128] row-major.
template <typename T>
__global__ void __launch_bounds__(256)
per_block_cast_kernel(const T* __restrict__ w, uint8_t* __restrict__ q, float* __restrict__ scales, int n, int k) {
    __shared__ float wave_max[4];
    const int k_blocks = k / 128;
    const int kb = blockIdx.x % k_blocks, nb = blockIdx.x / k_blocks;
    const int part = threadIdx.x & 15, row_in_step = threadIdx.x >> 4;      // 16 rows per step, 8 steps
    F32x8 v[8];
    float amax = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const int row = nb * 128 + s * 16 + row_in_step;
        if (row < n) {
            v[s] = load8(w + static_cast<long long>(row) * k + kb * 128 + part * 8);
            amax = fmaxf(amax, abs_max8(v[s]));
        }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) amax = fmaxf(amax, __shfl_xor(amax, d, 64));
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3])), 1e-4f);
    const float factor = kFp8Max / amax;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const int row = nb * 128 + s * 16 + row_in_step;
        if (row < n)
            *reinterpret_cast<uint2*>(q + static_cast<long long>(row) * k + kb * 128 + part * 8) = quantise8(v[s], factor);
    }
    if (threadIdx.x == 0) scales[static_cast<long long>(nb) * k_blocks + kb] = amax / kFp8Max;
}

// x [m, k] -> q [m, k] e4m3, scales fp32 with element (i, kb) at i * stride_m + kb * stride_k.
template <typename T>
inline hipError_t launch_per_token_cast(const T* x, void* q, float* scales, long long stride_m, long long stride_k,
                                        int m, int k, hipStream_t stream) {
    if (m == 0 || k == 0) return hipSuccess;
    if (m < 0 || k < 0 || (k % 128) != 0 || stride_m < 0 || stride_k < 0) return hipErrorInvalidValue;
    if (!x || !q || !scales) return hipErrorInvalidValue;
    constexpr int UNROLL = 2;      // measured: 1 and 2 tie, 4 and 8 are slower (fewer workgroups in flight)
    const long long groups = static_cast<long long>(m) * (k / 128);
    const long long blocks = ceil_div<long long>(groups, 16 * UNROLL);
    if (blocks >= (1ll << 31)) return hipErrorInvalidValue;
    hipLaunchKernelGGL((per_token_cast_kernel<T, UNROLL>), dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, stream,
                       x, static_cast<uint8_t*>(q), scales, groups, k / 128, stride_m, stride_k);
    return hipGetLastError();
}

// w [n, k] -> q [n, k] e4m3, scales fp32 [ceil(n/128), k/128] row-major.
template <typename T>
inline hipError_t launch_per_block_cast(const T* w, void* q, float* scales, int n, int k, hipStream_t stream) {
    if (n == 0 || k == 0) return hipSuccess;
    if (n < 0 || k < 0 || (k % 128) != 0) return hipErrorInvalidValue;
    if (!w || !q || !scales) return hipErrorInvalidValue;
    const long long blocks = static_cast<long long>(ceil_div(n, 128)) * (k / 128);
    if (blocks >= (1ll << 31)) return hipErrorInvalidValue;
    hipLaunchKernelGGL((per_block_cast_kernel<T>), dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, stream,
                       w, static_cast<uint8_t*>(q), scales, n, k);
    return hipGetLastError();
}

} // namespace yan
