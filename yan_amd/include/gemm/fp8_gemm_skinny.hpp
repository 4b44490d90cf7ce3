// Block-scaled FP8 GEMM for a handful of activation rows (m <= 128): the decode shape, bound by streaming the
// weights out of HBM once, not by the matrix core.
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


// ---------------------------------------------------------------------------------------------------------------------
// Split-K variant for 17..64 activation rows (and the default decode path): there the kernel above spends its time
// re-reading the activations (every one of its N/16 workgroups reads all m*K bytes). Here a workgroup owns 64 weight rows
// and 1/S of K, so the activations are read N/64 times in all, and S * N/64 workgroups still fill the chip:
//   * the workgroup's activation slab (16*TM rows x up to 16 K blocks, <= 128 KB) is copied into LDS once, all copies
//     issued up front; its weight fragments go straight to registers, all loads issued up front as well: each CU has
//     its whole share of both operands in flight from the first microsecond;
//   * wave (na, kh) multiplies weight atom na (16 rows) by all TM activation atoms over half kh of the K blocks;
//   * the two K halves meet through LDS, then the S splits meet through a fp32 scratch buffer: every workgroup writes
//     its 64 x 16*TM partial tile, and the last one to arrive for a column tile (an atomic counter says who) adds the
//     S partials in split order, so the result does not depend on arrival order, and writes bf16.
// The scratch buffer and the counters belong to the library (allocated on first use, counters reset by the kernel
// itself); launches that overlap in time on one device would share them and must not be issued concurrently.
template <int SHAPE_N, int SHAPE_K, int TM, int KBS_MAX>
__global__ void __launch_bounds__(8 * kWaveSize)
fp8_gemm_splitk_kernel(const uint8_t* __restrict__ lhs, const float* __restrict__ lhs_scales,
                       const uint8_t* __restrict__ rhs, const float* __restrict__ rhs_scales,
                       __bf16* __restrict__ out, int m, int n_rt, int k_rt, int sa_stride_m, int sa_stride_k,
                       int kbs /* K blocks per split, <= KBS_MAX */, int splits, float* __restrict__ scratch,
                       unsigned* __restrict__ counters) {
    using Atom = MfmaFP8_16x16x128;
    constexpr int NW = 8, KH = KBS_MAX / 2, ROWS_A = 16 * TM;
    static_assert(KBS_MAX % 2 == 0 && KBS_MAX * ROWS_A * kRowBytes >= 4 * TM * kWaveSize * 16, "the K halves meet in the slab's LDS");
    const int N = SHAPE_N ? SHAPE_N : n_rt, K = SHAPE_K ? SHAPE_K : k_rt;
    const int NUM_K_BLOCKS = K / 128, NUM_N_BLOCKS = ceil_div(N, 128);

    __shared__ __attribute__((aligned(1024))) uint8_t lds_a[KBS_MAX * ROWS_A * kRowBytes];     // [kb][row][128]
    __shared__ __attribute__((aligned(16))) float lds_sa[KBS_MAX][16][TM];                     // [kb][col][atom]
    __shared__ unsigned arrival;

    const int n_tile = blockIdx.x / splits, split = blockIdx.x % splits;
    const int n0 = n_tile * 64, kb0 = split * kbs;
    const int kb_end = min(kb0 + kbs, NUM_K_BLOCKS);            // this split's K blocks: [kb0, kb_end)
    const int lane = get_lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const int na = wave % 4, kh = wave / 4;
    const int g = lane / 16, col = lane % 16;

    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(lhs, uint32_t(m) * K);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(rhs, uint32_t(N) * K);
    const uint32_t sa_bytes = (uint32_t(m - 1) * sa_stride_m + uint32_t(NUM_K_BLOCKS - 1) * sa_stride_k + 1) * 4;
    const __amdgpu_buffer_rsrc_t rsrc_sa = make_rsrc(lhs_scales, sa_bytes);

    // Activation slab -> LDS: one copy instruction moves 8 rows of one K block; instruction e = (kb, 8-row group).
    {
        constexpr int GROUPS = ROWS_A / 8;
        const int sub = lane >> 3, slot = lane & 7;
#pragma unroll
        for (int e0 = 0; e0 < KBS_MAX * GROUPS; e0 += NW) {
            const int e = e0 + wave;
            const int kbl = e / GROUPS, grp = e % GROUPS;
            const int row = grp * 8 + sub;
            const int logical = slot ^ swizzle_of_row(row);
            const bool valid = kb0 + kbl < kb_end;
            const uint32_t voff = valid ? uint32_t(row) * K + logical * kChunk : kOutOfRange;
            if ((KBS_MAX * GROUPS) % NW == 0 || e < KBS_MAX * GROUPS)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, YAN_LDS_PTR(lds_a + (kbl * ROWS_A + grp * 8) * kRowBytes), kChunk,
                                                         voff, (kb0 + kbl) * kRowBytes, 0, 0);
        }
    }
    // Weight fragments of this wave's K blocks -> registers, everything in flight at once.
    const int kw0 = kb0 + kh * KH;                                // this wave's K blocks: [kw0, kw0 + KH) within the split
    const uint32_t voff_b = uint32_t(n0 + na * 16 + col) * K + 32 * g;
    const float* sb_row = rhs_scales + size_t(min((n0 + na * 16) / 128, NUM_N_BLOCKS - 1)) * NUM_K_BLOCKS;
    i32x4 bq[KH][2];
    float sb[KH];
#pragma unroll
    for (int i = 0; i < KH; ++i) {
        const int kb = kw0 + i;
        const bool valid = kb < kb_end && kh * KH + i < kbs;
        const uint32_t vb = valid ? voff_b : kOutOfRange;
        bq[i][0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vb, kb * kRowBytes, 0);
        bq[i][1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vb, kb * kRowBytes + 16, 0);
        sb[i] = sb_row[min(kb, NUM_K_BLOCKS - 1)];
    }
    // Activation scales of the split, once per workgroup: thread -> (K block, row), parked as [kb][row % 16][row / 16].
    for (int e = threadIdx.x; e < KBS_MAX * ROWS_A; e += NW * kWaveSize) {
        const int kbl = e / ROWS_A, row = e % ROWS_A;
        const int kbc = min(kb0 + kbl, NUM_K_BLOCKS - 1);
        lds_sa[kbl][row % 16][row / 16] = buffer_load_f32(rsrc_sa, uint32_t(row) * sa_stride_m * 4, kbc * sa_stride_k * 4);
    }

    wait_for_copies();
    __syncthreads();

    f32x4 acc[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int off0 = frag_offset<16>(lane, 2 * g), off1 = frag_offset<16>(lane, 2 * g + 1);
#pragma unroll
    for (int i = 0; i < KH; ++i) {
        const i32x8 bf = {bq[i][0][0], bq[i][0][1], bq[i][0][2], bq[i][0][3], bq[i][1][0], bq[i][1][1], bq[i][1][2], bq[i][1][3]};
        const uint8_t* slab = lds_a + (kh * KH + i) * ROWS_A * kRowBytes;
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            const i32x4 lo = *reinterpret_cast<const i32x4*>(slab + j * 16 * kRowBytes + off0);
            const i32x4 hi = *reinterpret_cast<const i32x4*>(slab + j * 16 * kRowBytes + off1);
            const i32x8 af = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            const f32x4 p = Atom::mma(bf, af, f32x4{0.f, 0.f, 0.f, 0.f});
            const float scale = lds_sa[kh * KH + i][col][j] * sb[i];
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[j][r] = __builtin_fmaf(p[r], scale, acc[j][r]);
        }
    }

    // The two K halves of a weight atom meet in LDS (the slab is no longer needed); the lower half's wave carries on.
    __syncthreads();
    float (*halves)[TM][kWaveSize][4] = reinterpret_cast<float (*)[TM][kWaveSize][4]>(lds_a);
    if (kh == 1) {
#pragma unroll
        for (int j = 0; j < TM; ++j) *reinterpret_cast<f32x4*>(halves[na][j][lane]) = acc[j];
    }
    __syncthreads();
    // scratch layout: [n_tile][split][atom j][weight atom na][lane][4 floats]. The partials cross between XCDs, whose
    // L2s do not see each other's lines: they are written through to memory and read back past the caches (device-
    // scope cache bits on the accesses themselves), which costs nothing next to a device-scope fence, which on this
    // part writes back and invalidates a whole L2.
    constexpr int kDeviceScope = 1 | 16;                          // sc0 | sc1
    constexpr int kTileFloats = TM * 4 * kWaveSize * 4;
    const __amdgpu_buffer_rsrc_t rsrc_sc = make_rsrc(scratch + size_t(n_tile) * splits * kTileFloats, uint32_t(splits) * kTileFloats * 4);
    if (kh == 0) {
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            acc[j] += *reinterpret_cast<const f32x4*>(halves[na][j][lane]);
            if (splits > 1)
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, acc[j]), rsrc_sc,
                                                       ((j * 4 + na) * kWaveSize + lane) * 16, split * kTileFloats * 4, kDeviceScope);
        }
    }
    if (splits > 1) {
        wait_for_copies();                                        // the write-through stores have been acknowledged
        __syncthreads();
        if (threadIdx.x == 0) arrival = atomicAdd(&counters[n_tile], 1u);
        __syncthreads();
        if (arrival != unsigned(splits - 1)) return;          // someone else finishes this column tile
        if (threadIdx.x == 0) counters[n_tile] = 0;           // ready for the next launch
    }
    if (kh == 0) {
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            f32x4 sum = acc[j];
            if (splits > 1) {
                sum = f32x4{0.f, 0.f, 0.f, 0.f};
                for (int s = 0; s < splits; ++s)
                    sum += __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                               rsrc_sc, ((j * 4 + na) * kWaveSize + lane) * 16, s * kTileFloats * 4, kDeviceScope));
            }
            const int mm = j * 16 + col, nn = n0 + na * 16 + 4 * g;
            if (mm < m && nn < N) *reinterpret_cast<bf16x4*>(out + size_t(mm) * N + nn) = pack4(sum, __bf16{});
        }
    }
}

// Library-owned scratch for the split-K meeting point: grown on demand, kept until the process ends.
struct SplitKScratch {
    float*    partials = nullptr;
    unsigned* counters = nullptr;
    size_t    partial_bytes = 0, counter_count = 0;
    int       device = -1;

    hipError_t reserve(size_t bytes, size_t count) {
        int dev = 0;
        if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
        if (dev != device) { partials = nullptr; counters = nullptr; partial_bytes = 0; counter_count = 0; device = dev; }   // one device at a time
        if (bytes > partial_bytes) {
            if (partials) (void)hipFree(partials);
            partials = nullptr; partial_bytes = 0;
            if (hipError_t e = hipMalloc(reinterpret_cast<void**>(&partials), bytes); e != hipSuccess) return e;
            partial_bytes = bytes;
        }
        if (count > counter_count) {
            if (counters) (void)hipFree(counters);
            counters = nullptr; counter_count = 0;
            if (hipError_t e = hipMalloc(reinterpret_cast<void**>(&counters), count * sizeof(unsigned)); e != hipSuccess) return e;
            if (hipError_t e = hipMemset(counters, 0, count * sizeof(unsigned)); e != hipSuccess) return e;
            counter_count = count;
        }
        return hipSuccess;
    }
};

inline SplitKScratch& splitk_scratch() {
    static SplitKScratch scratch;
    return scratch;
}

// K blocks per split and number of splits for n weight rows and k depth on `num_cus` compute units, `wgs_per_cu`
// workgroups resident per unit, at most `kbs_max` K blocks per split (the LDS slab). Every candidate split count is
// priced as rounds of workgroups times (K blocks per workgroup + a fixed cost of about 6 blocks for launch, meeting
// and tail) and the cheapest wins: it fills the chip once where it can and never spills a few workgroups into a
// second round.
inline void splitk_plan(int n, int k, int num_cus, int kbs_max, int wgs_per_cu, int* kbs, int* splits) {
    const int nkb = k / 128, n_tiles = ceil_div(n, 64), slots = num_cus * wgs_per_cu;
    int best_cost = 1 << 30;
    for (int s = ceil_div(nkb, kbs_max); s <= nkb; ++s) {
        const int per_split = ceil_div(nkb, s), used = ceil_div(nkb, per_split);
        if (used != s) continue;                            // the same work with fewer workgroups was priced already
        const int cost = ceil_div(n_tiles * s, slots) * (per_split + 6);
        if (cost < best_cost) { best_cost = cost; *kbs = per_split; *splits = s; }
    }
}

template <int SHAPE_N, int SHAPE_K, int TM, int KBS_MAX = 8>
inline hipError_t launch_fp8_splitk(__hip_bfloat16* out, const void* lhs, const float* lhs_scales, int lhs_scales_stride_m,
                                    int lhs_scales_stride_k, const void* rhs, const float* rhs_scales, int m, int n, int k,
                                    hipStream_t stream, int num_cus) {
    if (m == 0 || n == 0) return hipSuccess;
    if (m < 0 || m > 16 * TM || n < 0 || k <= 0 || (n % 4) != 0 || (k % 128) != 0 || num_cus <= 0) return hipErrorInvalidValue;
    if ((SHAPE_N && n != SHAPE_N) || (SHAPE_K && k != SHAPE_K)) return hipErrorInvalidValue;
    if (!out || !lhs || !lhs_scales || !rhs || !rhs_scales) return hipErrorInvalidValue;
    if (uint64_t(16 * TM) * k >= kOutOfRange || (uint64_t(n) + 64) * k >= kOutOfRange) return hipErrorInvalidValue;
    int kbs = 0, splits = 0;
    splitk_plan(n, k, num_cus, KBS_MAX, KBS_MAX <= 8 ? 2 : 1, &kbs, &splits);
    if (kbs > KBS_MAX) return hipErrorInvalidValue;
    const int n_tiles = ceil_div(n, 64);
    SplitKScratch& sc = splitk_scratch();
    if (splits > 1)
        if (hipError_t e = sc.reserve(size_t(n_tiles) * splits * TM * 4 * kWaveSize * 4 * sizeof(float), size_t(n_tiles)); e != hipSuccess) return e;
    hipLaunchKernelGGL((fp8_gemm_splitk_kernel<SHAPE_N, SHAPE_K, TM, KBS_MAX>), dim3(n_tiles * splits), dim3(8 * kWaveSize), 0, stream,
                       static_cast<const uint8_t*>(lhs), lhs_scales, static_cast<const uint8_t*>(rhs), rhs_scales,
                       reinterpret_cast<__bf16*>(out), m, n, k, lhs_scales_stride_m, lhs_scales_stride_k, kbs, splits,
                       sc.partials, sc.counters);
    return hipGetLastError();
}

} // namespace yan
