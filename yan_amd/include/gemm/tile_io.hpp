// Moving K-major operand tiles HBM -> LDS -> MFMA fragments on gfx950, and writing accumulators back.
//
// Both GEMMs in this directory stage tiles whose rows are 128 bytes along K (64 bf16 or 128 e4m3 values).
// This file is what stands in for the reference's TMA descriptors and swizzled shared-memory layouts
// (yan/include/gemm/fp8_gemm.cuh:55-113, yan/include/gemm/cute_gemm.cuh:278-316).
//
// HBM -> LDS: `buffer_load_dwordx4 ... lds`. One wave instruction moves 64 x 16 bytes and the hardware places
// lane i's 16 bytes at LDS address M0 + 16*i, i.e. one instruction fills 8 consecutive tile rows. The LDS side
// is therefore fixed; the swizzle is applied on the global side by choosing WHICH 16-byte chunk of the row
// each lane fetches. Rows past the end of the matrix get an offset beyond the descriptor's num_records, for
// which the hardware returns zeros, so tails need no branches.
//
// LDS layout: row r of a tile starts at byte 128*r; its logical chunk c (16 bytes) sits in slot
// c ^ swizzle_of_row(r). An MFMA operand read has lanes of consecutive rows fetch the same logical chunk; the
// XOR spreads any 8 consecutive rows over the 8 slots and rows r, r+8 over different slots, so neither a
// 32-bank nor a 64-bank LDS sees a conflict for ds_read_b128.
#pragma once

#include "utils.hpp"
#include "mfma_utils.hpp"

namespace yan {

__device__ __forceinline__ int swizzle_of_row(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// Offsets at or above this fail the bounds check of every descriptor this code builds (all < 2 GiB).
constexpr uint32_t kOutOfRange = 0x80000000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

// Block until every copy this wave has started (and every other vector-memory load) has landed. A workgroup
// barrier alone is not enough before reading a staged tile: the compiler's fence in __syncthreads() only waits
// for as many outstanding vector-memory operations as its memory model needs, and it does not count copies into
// LDS among them.
__device__ __forceinline__ void wait_for_copies() {
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, kNoWaitLgkm));
}

// One fp32 through a descriptor: per-lane byte offset + wave-uniform byte offset; out of range reads 0.0f.
__device__ __forceinline__ float buffer_load_f32(__amdgpu_buffer_rsrc_t rsrc, uint32_t voffset, uint32_t soffset) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, voffset, soffset, 0));
}

// Output stores through a descriptor, with or without the non-temporal hint (cache policy bit 1 on gfx950), chosen at
// run time. Two intrinsic calls with different immediates on purpose: a pair of ordinary stores that differ only in
// their non-temporal metadata is merged by the compiler into one plain store.
__device__ __forceinline__ void buffer_store_16(i32x4 v, __amdgpu_buffer_rsrc_t rsrc, uint32_t voffset, bool streaming) {
    if (streaming) __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, voffset, 0, 2);
    else __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, voffset, 0, 0);
}
template <typename T8>      // any 8-byte vector
__device__ __forceinline__ void buffer_store_8(T8 v, __amdgpu_buffer_rsrc_t rsrc, uint32_t voffset, bool streaming) {
    typedef int i32x2 __attribute__((ext_vector_type(2)));
    static_assert(sizeof(T8) == 8);
    if (streaming) __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(i32x2, v), rsrc, voffset, 0, 2);
    else __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(i32x2, v), rsrc, voffset, 0, 0);
}
// Descriptor over an output tile whose first element is `origin`: offsets are relative to it, bounds are the caller's
// business (rows and columns past the matrix are skipped by predicate).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_out_rsrc(const void* origin) { return make_rsrc(origin, 0xffffffffu); }

// Per-thread state for staging a ROWS x 128-byte tile with NUM_WAVES waves: one VGPR. Everything that varies
// per pass or per k-tile is wave-uniform and rides in the instruction's scalar offset, which the hardware adds
// before its bounds check; a row past the end of the matrix lands at or beyond num_records and reads as zero.
template <int ROWS, int NUM_WAVES>
struct TileStager {
    static_assert(ROWS % 16 == 0 && NUM_WAVES % 2 == 0);
    static constexpr int GROUPS = ROWS / 8;                       // 8-row groups, one instruction each
    static constexpr int PASSES = ceil_div(GROUPS, NUM_WAVES);
    // Every wave issues every pass, so that the steady state of a k-loop has no wave-dependent branch and every wave
    // has the same number of copies in flight. A wave whose group lies past the tile (only possible in the last
    // pass) is sent out of range and moves zeros into rows ROWS .. PADDED_ROWS - 1, which the LDS tile must have.
    static constexpr int PADDED_ROWS = PASSES * NUM_WAVES * 8;

    uint32_t voff;        // byte offset of this lane's chunk for pass 0 at K = 0
    uint32_t pass_pitch;  // bytes between the rows of consecutive passes (uniform)
    int      logical;     // logical chunk index this lane fetches

    // The tile starts at matrix row `tile_row0`; rows have a pitch of `ld_bytes`.
    __device__ __forceinline__ void init(int tile_row0, uint32_t ld_bytes, int wave, int lane) {
        const int sub = lane >> 3, slot = lane & 7;
        logical    = slot ^ sub ^ (wave & 1);     // == slot ^ swizzle_of_row(8*q + sub) for every q = wave (mod 2)
        voff       = uint32_t(tile_row0 + wave * 8 + sub) * ld_bytes + logical * kChunk;
        pass_pitch = uint32_t(NUM_WAVES * 8) * ld_bytes;
    }

    // Start the copy of the k-tile at byte `k_byte0` of every row into `lds_tile`.
    __device__ __forceinline__ void issue(__amdgpu_buffer_rsrc_t rsrc, uint8_t* lds_tile, int k_byte0, int wave) const {
        issue_from(rsrc, lds_tile, k_byte0, wave, voff);
    }

    // Lane offset to use for a last k-tile of which only `valid_bytes` (a multiple of 16) per row exist: lanes
    // whose chunk lies beyond the row end are sent out of range and move zeros.
    __device__ __forceinline__ uint32_t tail_voff(int valid_bytes) const {
        return logical * kChunk < valid_bytes ? voff : kOutOfRange;
    }

    // One pass (8 rows per wave) of the copy, for callers that interleave the passes with other work.
    __device__ __forceinline__ void issue_pass(__amdgpu_buffer_rsrc_t rsrc, uint8_t* lds_tile, int k_byte0, int wave, int j) const {
        issue_pass_from(rsrc, lds_tile, k_byte0, wave, j, voff);
    }

    __device__ __forceinline__ void issue_pass_from(__amdgpu_buffer_rsrc_t rsrc, uint8_t* lds_tile, int k_byte0, int wave, int j,
                                                    uint32_t lane_voff) const {
        const int q = j * NUM_WAVES + wave;
        const uint32_t past_tile = (GROUPS % NUM_WAVES == 0 || q < GROUPS) ? 0u : kOutOfRange;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, YAN_LDS_PTR(lds_tile + q * 8 * kRowBytes), kChunk, lane_voff | past_tile,
                                                 k_byte0 + j * pass_pitch, 0, 0);
    }

    __device__ __forceinline__ void issue_from(__amdgpu_buffer_rsrc_t rsrc, uint8_t* lds_tile, int k_byte0, int wave,
                                               uint32_t lane_voff) const {
#pragma unroll
        for (int j = 0; j < PASSES; ++j) {
            const int q = j * NUM_WAVES + wave;
            const uint32_t past_tile = (GROUPS % NUM_WAVES == 0 || q < GROUPS) ? 0u : kOutOfRange;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, YAN_LDS_PTR(lds_tile + q * 8 * kRowBytes), kChunk,
                                                     lane_voff | past_tile, k_byte0 + j * pass_pitch, 0, 0);
        }
    }
};

// Where the SPLIT_K parts of a split-K tile meet (fp8_gemm.hpp, bf16_gemm.hpp). Wave w of every part leaves its VECS
// 16-byte vectors of sums in `partials` (laid out as the registers are: part, wave, vector, lane) and counts itself in at
// counters[tile * NW + w]; the wave that arrives last adds the parts up in the order of their K ranges, whichever it was
// itself, puts the counter back to zero for the next launch and returns true: it stores the tile. The counters must be zero
// before the first launch. `sums(v)` is a reference to vector v of the caller's accumulators.
// The parts run on different XCDs, whose L2s do not see each other's lines. The sums are therefore written and read at
// device scope (cache policy sc1: written through to memory, read from there), as the counter is; a device-scope fence
// instead would write back and invalidate the whole L2 of the XCD once per wave (measured: 45-110 us for a 10 us GEMM).
template <int SPLIT_K, int NW, int VECS, typename Sums>
__device__ __forceinline__ bool
meet_partials(Sums&& sums, float* __restrict__ partials, unsigned* __restrict__ counters, int tile_slot, int split, int wave, int lane) {
    constexpr int kDeviceScope = 16;        // cache-policy bit sc1 of gfx950 buffer instructions
    constexpr uint32_t VEC_BYTES = kWaveSize * 16, WAVE_BYTES = VECS * VEC_BYTES, PART_BYTES = NW * WAVE_BYTES;
    const __amdgpu_buffer_rsrc_t parts = make_rsrc(partials + size_t(tile_slot) * (SPLIT_K * PART_BYTES / 4), SPLIT_K * PART_BYTES);
    const uint32_t lane_off = uint32_t(wave) * WAVE_BYTES + lane * 16;
#pragma unroll
    for (int v = 0; v < VECS; ++v)
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, f32x4(sums(v))), parts, lane_off + v * VEC_BYTES, split * PART_BYTES, kDeviceScope);
    // the sums have reached memory before the count is taken
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, kNoWaitLgkm));
    asm volatile("" ::: "memory");
    unsigned before = 0;
    if (lane == 0) before = __hip_atomic_fetch_add(counters + tile_slot * NW + wave, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    before = __builtin_amdgcn_readfirstlane(before);
    asm volatile("" ::: "memory");
    if (before != SPLIT_K - 1) return false;
#pragma unroll
    for (int v = 0; v < VECS; ++v) sums(v) = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < SPLIT_K; ++s)
#pragma unroll
        for (int v = 0; v < VECS; ++v)
            sums(v) += __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(parts, lane_off + v * VEC_BYTES, s * PART_BYTES, kDeviceScope));
    if (lane == 0) __hip_atomic_store(counters + tile_slot * NW + wave, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return true;
}

// Puts the arrival counters at the start of a split-K workspace back to zero: what a caller does once for a fresh
// workspace, and again after anything that may have left a launch half done (a launch that reported an error, launches
// that overlapped on one workspace). A fill kernel rather than a memset node, so the call may be captured into a graph.
template <int = 0>      // a template so that only code that launches it carries it
__global__ void __launch_bounds__(256) split_k_reset_kernel(unsigned* __restrict__ counters, int count) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < count) __hip_atomic_store(counters + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int V = 0>
inline hipError_t launch_split_k_reset(void* workspace, size_t counter_bytes, hipStream_t stream) {
    if (!workspace) return hipErrorInvalidValue;
    const int count = int(counter_bytes / 4);
    hipLaunchKernelGGL(split_k_reset_kernel<V>, dim3(ceil_div(count, 256)), dim3(256), 0, stream, static_cast<unsigned*>(workspace), count);
    return hipGetLastError();
}

// Byte offset, relative to the first row of an R-row atom that starts at a multiple of 16 tile rows, of logical
// chunk `chunk` of the row this lane owns.
template <int R>
__device__ __forceinline__ int frag_offset(int lane, int chunk) {
    const int i = lane % R;
    return i * kRowBytes + ((chunk ^ swizzle_of_row(i)) * kChunk);
}

// fp32 -> bf16 / f16, round to nearest even, four at a time.
__device__ __forceinline__ bf16x4 pack4(f32x4 v, __bf16) { return __builtin_convertvector(v, bf16x4); }
__device__ __forceinline__ f16x4  pack4(f32x4 v, _Float16) { return __builtin_convertvector(v, f16x4); }

} // namespace yan
