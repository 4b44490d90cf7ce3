// Dense 16-bit GEMM for a handful of activation rows (the launcher sends m <= 16 * TM here): bound by streaming the weights
// out of HBM once, not by the matrix core.
//
// Same contract as bf16_gemm.hpp (c[m,n] = a[m,k] @ b[n,k]^T, fp32 accumulate; yan/jit_kernels/cute_gemm.py:21-64), a
// different kernel: the tiled kernels give a workgroup at least 64 weight rows, so a problem with few thousand of them
// puts a quarter of the compute units to work and each of those pulls at the rate one compute unit can
// (64 x 4096 x 7168: 64 tiles, 2.2 TB/s of weights). Here, as in fp8_gemm_skinny.hpp:
//   * one workgroup per 16 weight rows (n/16 workgroups: 256 for n = 4096), every CU pulling its own slice of B;
//   * no LDS staging and no barriers in the main loop: wave w of a workgroup owns the 128-byte K blocks w, w+W, w+2W, ...
//     and streams their operand fragments straight into registers, DEPTH blocks ahead;
//   * per K block two 16x16x32 MFMAs per 16 activation rows: lane group g holds bytes [32g, 32g+32) of its row, i.e. chunks
//     2g and 2g+1, for both operands, so the first MFMA contracts over the even chunks and the second over the odd ones;
//   * the W partial sums of a workgroup meet once, through LDS, and leave as bf16 / fp16.
// The activations are re-read from L2 by every workgroup (m * k * 2 bytes each).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "utils.hpp"
#include "mfma_utils.hpp"
#include "tile_io.hpp"

namespace yan {

// TM: 16-row activation atoms covered (m <= 16*TM). NUM_WAVES: waves sharing the K blocks of one workgroup.
template <typename Atom, typename Elem, int TM, int NUM_WAVES>
__global__ void __launch_bounds__(NUM_WAVES * kWaveSize)
dense_gemm_skinny_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, Elem* __restrict__ C, int m, int n, int k) {
    using Frag = typename Atom::Frag;
    static_assert(Atom::R == 16 && sizeof(Frag) == 16 && sizeof(Elem) == 2);
    constexpr int DEPTH = TM <= 2 ? 6 : 4;          // K blocks in flight per wave
    static_assert(NUM_WAVES >= TM, "the final reduction gives one activation atom to each of the first TM waves");
    const int k_bytes = k * 2, num_k_blocks = k_bytes / kRowBytes;

    __shared__ __attribute__((aligned(16))) float partial[NUM_WAVES][TM][kWaveSize][4];

    const int n0 = blockIdx.x * 16;
    const int lane = get_lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const int g = lane / 16, col = lane % 16;

    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(A, uint32_t(m) * k_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(B, uint32_t(n) * k_bytes);
    // Lane (col, g) holds bytes [32g, 32g+32) of K block kb of row `col` of its atom, for both operands; rows past the end
    // of either matrix start beyond num_records and read as zero.
    const uint32_t voff_b = uint32_t(n0 + col) * k_bytes + 32 * g;
    const uint32_t voff_a = uint32_t(col) * k_bytes + 32 * g;

    // Every workgroup reads all of the activations: starting each at a different K block (and wrapping around) spreads
    // the requests over the whole activation matrix instead of queueing them on the same few cache lines.
    const int rot = (blockIdx.x * 7) % num_k_blocks;
    auto rotated = [&](int kb) { const int r = kb + rot; return r >= num_k_blocks ? r - num_k_blocks : r; };

    struct Stage {
        i32x4 b[2];
        i32x4 a[TM][2];
    };
    Stage st[DEPTH];
    auto load = [&](Stage& s, int seq) {
        const bool valid = seq < num_k_blocks;          // past the end: operands read as zero
        const uint32_t vb = valid ? voff_b : kOutOfRange, va = valid ? voff_a : kOutOfRange;
        const int kb = rotated(min(seq, num_k_blocks - 1));
        s.b[0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vb, kb * kRowBytes, 0);
        s.b[1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vb, kb * kRowBytes + 16, 0);
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            s.a[j][0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, va, kb * kRowBytes + j * 16 * k_bytes, 0);
            s.a[j][1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, va, kb * kRowBytes + j * 16 * k_bytes + 16, 0);
        }
    };

    f32x4 acc[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
    for (int s = 0; s < DEPTH; ++s) load(st[s], wave + s * NUM_WAVES);
    for (int kb = wave; kb < num_k_blocks; kb += DEPTH * NUM_WAVES) {
#pragma unroll
        for (int s = 0; s < DEPTH; ++s) {
            const Stage& c = st[s];
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                acc[j] = Atom::mma(__builtin_bit_cast(Frag, c.b[0]), __builtin_bit_cast(Frag, c.a[j][0]), acc[j]);
                acc[j] = Atom::mma(__builtin_bit_cast(Frag, c.b[1]), __builtin_bit_cast(Frag, c.a[j][1]), acc[j]);
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
        if (mm < m && nn < n) *reinterpret_cast<decltype(pack4(sum, Elem{}))*>(C + size_t(mm) * n + nn) = pack4(sum, Elem{});
    }
}

// Whether the weight-streaming kernel can run a problem at all: whole 128-byte K blocks, 8-byte output runs.
__host__ __device__ constexpr bool dense_skinny_fits(int m, int n, int k, int tm) {
    return m > 0 && m <= 16 * tm && n > 0 && (n % 4) == 0 && k > 0 && (k % 64) == 0;
}

// Launcher for m <= 16*TM. Returns hipErrorInvalidValue for sizes outside the kernel's reach.
template <typename Atom, typename Elem, int TM, int NUM_WAVES>
inline hipError_t launch_dense_skinny(int m, int n, int k, const void* a, const void* b, void* c, hipStream_t stream) {
    if (m == 0 || n == 0) return hipSuccess;
    if (!dense_skinny_fits(m, n, k, TM) || !a || !b || !c) return hipErrorInvalidValue;
    if (uint64_t(16 * TM) * k * 2 >= kOutOfRange || (uint64_t(n) + 16) * k * 2 >= kOutOfRange) return hipErrorInvalidValue;
    hipLaunchKernelGGL((dense_gemm_skinny_kernel<Atom, Elem, TM, NUM_WAVES>), dim3(ceil_div(n, 16)), dim3(NUM_WAVES * kWaveSize), 0,
                       stream, static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b), static_cast<Elem*>(c), m, n, k);
    return hipGetLastError();
}

} // namespace yan
