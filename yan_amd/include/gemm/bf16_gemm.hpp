// C[m,n] = A[m,k] . B[n,k]^T for bf16 (or fp16) operands, fp32 accumulation, gfx950.
//
// Entry point `gemm_tn<BLOCK_M, BLOCK_N, NUM_STAGES>` keeps the signature and layout contract of the
// reference's launcher (yan/include/gemm/cute_gemm.cuh:262-378: A [m,k] and B [n,k] row-major with K
// contiguous, C [m,n] row-major written in place, work enqueued on `stream`), but none of its structure:
// the reference kernel (cute_gemm.cuh:14-260) is a 128x128x32 cp.async/ldmatrix/mma.sync pipeline with fp16
// accumulation and no bounds handling. Here:
//   * macro tile BLOCK_M x BLOCK_N x 64 (128-byte rows), staged HBM -> LDS with buffer_load ... lds (tile_io.hpp);
//   * tiles of 256 rows and 160 to 256 columns: two LDS stages, 8 waves (two per SIMD), each with a (BLOCK_N/2) x 64 slab
//     of 16x16x32 MFMAs (128 accumulator registers for the 256-wide tile, tied to their instructions so that they stay
//     where they are); while one wave of a SIMD issues copies or waits for a fragment the other keeps the matrix core
//     busy, and the barrier between two k-tiles sits two steps before the end of the first, so that every wave still
//     holds work when it has passed it; one workgroup per compute unit walks the tiles (dense_gemm_body_8w);
//   * the smaller tiles (256 x 128 down to 64 x 64, widths of 64, 128, 192 and 256), which run problems bound by operand
//     streaming: a ring of three to eight LDS stages, 4 waves, one per SIMD, each with a (BLOCK_N/WAVES_N) x
//     (BLOCK_M/WAVES_M) slab of 32x32x16 MFMAs, up to 128 x 128 (256 accumulator registers, which the compiler keeps in
//     AGPRs) (dense_gemm_body);
//   * problems with long K and fewer ring tiles than compute units split K over SPLIT_K workgroups per tile, which meet in a
//     caller-provided workspace (dense_gemm_split_k, dense_meet_partials; 64 x 4096 x 7168: 64 workgroups of 64 x 64 become 256);
//   * B rows feed the MFMA row operand and A rows the column operand, so a lane's four consecutive accumulator
//     registers are four consecutive n of one m: contiguous in C;
//   * fp32 accumulators, round-to-nearest-even on the way out;
//   * any m and n (n % 4 == 0), k % 8 == 0; rows beyond m / n and the k tail read as zero.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "utils.hpp"
#include "mfma_utils.hpp"
#include "scheduler.hpp"
#include "tile_io.hpp"
#include "bf16_gemm_skinny.hpp"

namespace yan {

template <int BLOCK_M, int BLOCK_N>
struct DenseTileConfig {
    static constexpr int NUM_WAVES = 4;
    // A slab of at most 128 x 128 outputs: 256 accumulator registers per lane, out of the 512 a lone wave may hold.
    static constexpr int WAVES_N   = pick_waves_n(BLOCK_M, BLOCK_N, NUM_WAVES, 32, 128 * 128);
    static_assert(WAVES_N > 0, "no wave layout fits this tile");
    static constexpr int WAVES_M   = NUM_WAVES / WAVES_N;
    static constexpr int WTN = BLOCK_N / WAVES_N, WTM = BLOCK_M / WAVES_M;
    static_assert(WTN % 32 == 0 && WTM % 32 == 0, "wave slab must be a whole number of 32x32 atoms");
    static constexpr int LDS_BYTES = 2 * (BLOCK_M + BLOCK_N) * kRowBytes;
    static_assert(LDS_BYTES <= 160 * 1024, "two stages must fit the 160 KB LDS");
    // Deepest ring of LDS stages the 160 KB hold for this tile (at most 8); 2 for the 256 x 256 tile.
    static constexpr int STAGE_BYTES = (BLOCK_M + BLOCK_N) * kRowBytes;
    static constexpr int MAX_STAGES  = 160 * 1024 / STAGE_BYTES < 8 ? 160 * 1024 / STAGE_BYTES : 8;
};

// STAGES (3 ..): a ring of that many LDS stages with STAGES - 1 k-tiles in
// flight, for the smaller tiles, which are picked when a problem is bound by streaming its operands.
// Where the SPLIT_K parts of a dense tile meet (meet_partials in tile_io.hpp): the wave's TN x TM atoms of 16 sums each, as
// four 16-byte vectors per atom.
template <typename Acc>
struct AccQuarter {         // registers 4q .. 4q+3 of an accumulator, readable and writable as one f32x4
    Acc& acc;
    int  q;
    __device__ __forceinline__ operator f32x4() const { return f32x4{acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]}; }
    __device__ __forceinline__ void operator=(f32x4 v) const {
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[4 * q + r] = v[r];
    }
    __device__ __forceinline__ void operator+=(f32x4 v) const {
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[4 * q + r] += v[r];
    }
};
template <int SPLIT_K, int NW, int TN, int TM, typename Acc>
__device__ __forceinline__ bool
dense_meet_partials(Acc (&acc)[TN][TM], float* __restrict__ partials, unsigned* __restrict__ counters, int tile_slot, int split, int wave, int lane) {
    return meet_partials<SPLIT_K, NW, TN * TM * 4>([&](int v) { return AccQuarter<Acc>{acc[(v / 4) / TM][(v / 4) % TM], v % 4}; }, partials, counters,
                                                   tile_slot, split, wave, lane);
}

template <typename Atom, typename Elem, int BLOCK_M, int BLOCK_N, int STAGES, int SPLIT_K = 1>
__device__ __forceinline__ void
dense_gemm_body(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, Elem* __restrict__ C,
                int m, int n, int k, int bid, float* __restrict__ partials = nullptr, unsigned* __restrict__ counters = nullptr) {
    using Cfg = DenseTileConfig<BLOCK_M, BLOCK_N>;
    constexpr int NW = Cfg::NUM_WAVES, TN = Cfg::WTN / 32, TM = Cfg::WTM / 32;
    static_assert(STAGES >= 3 && STAGES <= Cfg::MAX_STAGES, "a ring of three or more stages that fits the LDS");
    // SPLIT_K > 1: launch slot `bid` is part `bid % SPLIT_K` of tile slot `bid / SPLIT_K`
    [[maybe_unused]] int split = 0;
    if constexpr (SPLIT_K > 1) { split = bid % SPLIT_K; bid /= SPLIT_K; }

    const XcdTileScheduler<> sched(m, n, BLOCK_M, BLOCK_N);
    const TileCoord tile = sched.tile_of(bid);
    if (!tile.valid) return;
    const int m0 = tile.m_idx * BLOCK_M, n0 = tile.n_idx * BLOCK_N;

    const int lane = get_lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const int wn = wave % Cfg::WAVES_N, wm = wave / Cfg::WAVES_N;

    const uint32_t ld_bytes = uint32_t(k) * 2;
    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(A, uint32_t(m) * ld_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(B, uint32_t(n) * ld_bytes);
    TileStager<BLOCK_M, NW> stage_a;
    TileStager<BLOCK_N, NW> stage_b;
    stage_a.init(m0, ld_bytes, wave, lane);
    stage_b.init(n0, ld_bytes, wave, lane);

    // k-tiles: `num_k_tiles` in all, the last one possibly partial (only `tail_bytes` of each row exist).
    const int k_bytes = k * 2;
    const int num_k_tiles = ceil_div(k_bytes, kRowBytes);
    const int tail_tile = (k_bytes % kRowBytes) ? num_k_tiles - 1 : -1;
    const uint32_t tail_a = stage_a.tail_voff(k_bytes % kRowBytes), tail_b = stage_b.tail_voff(k_bytes % kRowBytes);
    // this part's k-tiles; copies past them keep the count of instructions in flight and move nothing
    int kt_lo = 0, kt_hi = num_k_tiles;
    if constexpr (SPLIT_K > 1) {
        const int per = ceil_div(num_k_tiles, SPLIT_K);
        kt_lo = min(split * per, num_k_tiles);
        kt_hi = min(kt_lo + per, num_k_tiles);
    }
    const __amdgpu_buffer_rsrc_t rsrc_none = make_rsrc(A, 0);
    using StA = TileStager<BLOCK_M, NW>;
    using StB = TileStager<BLOCK_N, NW>;
    constexpr int NUM_COPIES = StA::PASSES + StB::PASSES;
    static_assert(StA::PADDED_ROWS == BLOCK_M && StB::PADDED_ROWS == BLOCK_N, "tiles are whole copy passes");
    // Copy number `d` (A passes first, then B passes) of k-tile `kt` into the given stage.
    auto copy_pass = [&](int d, int kt, uint8_t* la, uint8_t* lb) {
        const bool tail = kt == tail_tile;
        const bool live = kt < kt_hi;
        if (d < StA::PASSES) stage_a.issue_pass_from(live ? rsrc_a : rsrc_none, la, kt * kRowBytes, wave, d, tail ? tail_a : stage_a.voff);
        else stage_b.issue_pass_from(live ? rsrc_b : rsrc_none, lb, kt * kRowBytes, wave, d - StA::PASSES, tail ? tail_b : stage_b.voff);
    };

    // Lane-constant LDS offsets of the four 16-deep K steps inside a 64-deep tile.
    const int g = lane / 32;
    int koff[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) koff[kk] = frag_offset<32>(lane, 2 * kk + g);

    typename Atom::Acc acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // One k-tile = four 16-deep steps; the fragments of step kk+1 are fetched before the MFMAs of step kk issue.
    // `step_hook(kk)` runs once per step and is where the copies of the next k-tile are started.
    constexpr int SPREAD_STEPS = 2;
    auto copies_in_step = [](int kk) {
        int c = 0;
        for (int d = 0; d < NUM_COPIES; ++d) c += (d * SPREAD_STEPS / NUM_COPIES == kk);
        return c;
    };
    auto compute_tile = [&](const uint8_t* la, const uint8_t* lb, auto&& step_hook) {
        using Frag = typename Atom::Frag;
        const uint8_t* pa = la + wm * Cfg::WTM * kRowBytes;
        const uint8_t* pb = lb + wn * Cfg::WTN * kRowBytes;
        Frag nf[2][TN], mf[2][TM];
        auto fetch = [&](int kk) {
#pragma unroll
            for (int i = 0; i < TN; ++i) nf[kk & 1][i] = *reinterpret_cast<const Frag*>(pb + i * 32 * kRowBytes + koff[kk]);
#pragma unroll
            for (int j = 0; j < TM; ++j) mf[kk & 1][j] = *reinterpret_cast<const Frag*>(pa + j * 32 * kRowBytes + koff[kk]);
        };
        fetch(0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            step_hook(kk);
            if (kk + 1 < 4) fetch(kk + 1);
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int j = 0; j < TM; ++j) acc[i][j] = Atom::mma(nf[kk & 1][i], mf[kk & 1][j], acc[i][j]);
            // Issue order inside the step: one LDS read, one copy instruction, one MFMA, ... so that reads and
            // copies ride under the MFMAs instead of queueing in front of them.
            {
                constexpr int kDsRead = 0x100, kVmem = 0x020, kMfma = 0x008;
                const int reads = kk + 1 < 4 ? TN + TM : 0, copies = copies_in_step(kk);
#pragma unroll
                for (int x = 0; x < TN * TM; ++x) {
                    if (x < reads) __builtin_amdgcn_sched_group_barrier(kDsRead, 1, 0);
                    if (x < copies) __builtin_amdgcn_sched_group_barrier(kVmem, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // Ring: every wave issues NUM_COPIES copies per k-tile, in the same order, so "k-tile kt has landed" is "at
    // most (STAGES - 2) * NUM_COPIES of my copies are outstanding". The copies of k-tile kt + STAGES - 1 go to
    // the stage that was consumed in iteration kt - 1, which every wave has left once it is past the barrier.
    static_assert((BLOCK_M / 8) % NW == 0 && (BLOCK_N / 8) % NW == 0 && (STAGES - 2) * NUM_COPIES <= 63);
    constexpr int STAGE_BYTES = Cfg::STAGE_BYTES;
    __shared__ __attribute__((aligned(1024))) uint8_t ring[STAGES * STAGE_BYTES];
#pragma unroll
    for (int t = 0; t < STAGES - 1; ++t)
#pragma unroll
        for (int d = 0; d < NUM_COPIES; ++d) copy_pass(d, kt_lo + t, ring + t * STAGE_BYTES, ring + t * STAGE_BYTES + BLOCK_M * kRowBytes);
    int st = 0;
    for (int kt = kt_lo; kt < kt_hi; ++kt) {
        __builtin_amdgcn_s_waitcnt(waitcnt_imm((STAGES - 2) * NUM_COPIES, kNoWaitLgkm));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const uint8_t* cur = ring + st * STAGE_BYTES;
        uint8_t* nxt = ring + (st == 0 ? STAGES - 1 : st - 1) * STAGE_BYTES;
        compute_tile(cur, cur + BLOCK_M * kRowBytes, [&](int kk) {
#pragma unroll
            for (int d = 0; d < NUM_COPIES; ++d)
                if (d * SPREAD_STEPS / NUM_COPIES == kk) copy_pass(d, kt + STAGES - 1, nxt, nxt + BLOCK_M * kRowBytes);
        });
        st = st + 1 == STAGES ? 0 : st + 1;
    }

    // Epilogue: registers 4*q .. 4*q+3 of an atom are n = 8*q + 4*g + {0,1,2,3} of column m = lane % 32. Stored straight
    // from there a wave instruction writes 32 rows x 16 bytes; instead each wave turns its slab round through the
    // stage that was consumed last (the only one no copy is on its way into), 32 rows at a time, and stores 16 bytes
    // per lane in runs of 2 * WTN consecutive bytes per row. An output larger than the L2s together (8 x 4 MB) is
    // stored with the non-temporal hint, so that it does not push the operand panels out of them.
    const bool stream_out = size_t(m) * n * sizeof(Elem) > (size_t(32) << 20);
    const __amdgpu_buffer_rsrc_t rsrc_c = make_out_rsrc(C + size_t(m0) * n + n0);
    if constexpr (SPLIT_K > 1) {
        // every wave has read the last k-tile before any wave's epilogue writes into that stage
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoWaitVm, 0));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (!dense_meet_partials<SPLIT_K, NW>(acc, partials, counters, bid, split, wave, lane)) return;
    }
    constexpr int PITCH = Cfg::WTN * 2 + 16, REGION = 32 * PITCH;
    // lanes per row segment; rows one store instruction covers (a slab width that does not divide the wave leaves the last
    // lanes idle); store instructions per 32 rows
    constexpr int LANES_PER_ROW = Cfg::WTN / 8, ROWS_PER_STORE = kWaveSize / LANES_PER_ROW, STORES = ceil_div(32, ROWS_PER_STORE);
    static_assert(NW * REGION <= STAGE_BYTES && STORES >= 1 && sizeof(Elem) == 2);
    if ((n % 8) == 0) {
        // every wave has read the last k-tile (a bare barrier: nothing here depends on the copies still under way)
        if constexpr (SPLIT_K == 1) {
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoWaitVm, 0));
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        }
        uint8_t* region = ring + (st == 0 ? STAGES - 1 : st - 1) * STAGE_BYTES + wave * REGION;
        const int ml = lane % 32, r_in = lane / LANES_PER_ROW, c = lane % LANES_PER_ROW;
        const int n_in_tile = wn * Cfg::WTN + 8 * c;
#pragma unroll
        for (int j = 0; j < TM; ++j) {
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f32x4 v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                    *reinterpret_cast<decltype(pack4(v, Elem{}))*>(region + ml * PITCH + (32 * i + 8 * q + 4 * g) * 2) = pack4(v, Elem{});
                }
#pragma unroll
            for (int s = 0; s < STORES; ++s) {
                const int row = ROWS_PER_STORE * s + r_in, m_in_tile = wm * Cfg::WTM + 32 * j + row;
                const i32x4 v = *reinterpret_cast<const i32x4*>(region + row * PITCH + c * 16);
                if (r_in < ROWS_PER_STORE && row < 32 && m0 + m_in_tile < m && n0 + n_in_tile < n)
                    buffer_store_16(v, rsrc_c, uint32_t(m_in_tile * n + n_in_tile) * 2u, stream_out);
            }
        }
        return;
    }
    const int m_lane = m0 + wm * Cfg::WTM + lane % 32;
    const int n_lane = n0 + wn * Cfg::WTN + 4 * g;
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const int mm = m_lane + j * 32;
        if (mm >= m) continue;
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int nn = n_lane + i * 32 + q * 8;
                if (nn < n) {
                    const f32x4 v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                    buffer_store_8(pack4(v, Elem{}), rsrc_c, uint32_t((mm - m0) * n + nn - n0) * 2u, stream_out);
                }
            }
    }
}

// The same contraction with 8 waves (two per SIMD) and 16x16x32 atoms: each wave owns a (BLOCK_N/2) x (BLOCK_M/4) slab,
// 128 accumulator registers for the 256 x 256 tile. Two LDS stages. The kernel is persistent: a workgroup walks the tiles
// blockIdx.x, blockIdx.x + gridDim.x, ... (the launcher starts one workgroup per CU, or as many as the caller's cap
// allows), starts the copies of the next tile's first k-tile during the last k-tile of the current one, fetches that
// k-tile's first fragments before it turns to the epilogue, and its output stores drain while the next tile is already
// computing. With one workgroup per tile the drain and the first loads of every tile were exposed: 11 % of the time at
// 8192^3.
template <typename Atom, typename Elem, int BLOCK_M, int BLOCK_N>
__device__ __forceinline__ void
dense_gemm_body_8w(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, Elem* __restrict__ C, int m, int n, int k) {
    constexpr int NW = 8, WAVES_N = 2, WAVES_M = 4, WTN = BLOCK_N / WAVES_N, WTM = BLOCK_M / WAVES_M;
    constexpr int TN = WTN / 16, TM = WTM / 16, STEPS = 2 * TN;
    static_assert(WTN % 16 == 0 && WTM % 16 == 0 && TN * TM * 4 <= 128 && TN >= 4);
    using Frag = typename Atom::Frag;
    using StA = TileStager<BLOCK_M, NW>;
    using StB = TileStager<BLOCK_N, NW>;
    // BLOCK_N is any multiple of 32 from 128 to 256 (a problem whose tiles do not fill whole rounds of compute units with
    // one width often does with another); the weight tile in LDS is rounded up to whole copy passes of 64 rows.
    static_assert(StA::PADDED_ROWS == BLOCK_M, "the activation tile is whole copy passes");
    constexpr int LDS_ROWS_B = StB::PADDED_ROWS;
    constexpr int NUM_COPIES = StA::PASSES + StB::PASSES;

    const XcdTileScheduler<> sched(m, n, BLOCK_M, BLOCK_N, (long long)k * sizeof(Elem));
    const int num_slots = sched.grid_size();
    const int lane = get_lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const int wn = wave % WAVES_N, wm = wave / WAVES_N;
    const int g = lane / 16, col = lane % 16;

    const uint32_t ld_bytes = uint32_t(k) * 2;
    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(A, uint32_t(m) * ld_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(B, uint32_t(n) * ld_bytes);
    const int k_bytes = k * 2;
    const int num_k_tiles = ceil_div(k_bytes, kRowBytes);
    const int tail_tile = (k_bytes % kRowBytes) ? num_k_tiles - 1 : -1;
    // An output larger than the L2s together (8 x 4 MB) is stored with the non-temporal hint: kept in L2 it pushes
    // out the operand panels the other workgroups of the XCD are about to read (8192^3: 805 -> 754 us).
    const bool stream_out = size_t(m) * n * sizeof(Elem) > (size_t(32) << 20);

    // Every tile runs an even number of k-tiles, so that it starts in stage 0 and the stage of every k-step is known
    // at compile time (the compiler then sees that the copies into one stage cannot touch the fragments it reads from
    // the other, and does not wait for them): an odd count gets one more k-tile whose copies are sent out of range
    // and move zeros.
    const int k_tiles_run = (num_k_tiles + 1) & ~1;
    // What a wave needs to know of a tile to copy its k-tiles.
    struct TileIo {
        StA a;
        StB b;
        uint32_t tail_a, tail_b;
        int m0, n0;
        int k_rot;          // the k-tile this tile's walk over K starts at
        bool valid;
    };
    auto open_tile = [&](int slot) {
        TileIo t;
        const TileCoord coord = slot < num_slots ? sched.tile_of(slot) : TileCoord{0, 0, false};
        t.valid = coord.valid;
        t.m0 = coord.m_idx * BLOCK_M;
        t.n0 = coord.n_idx * BLOCK_N;
        t.a.init(t.m0, ld_bytes, wave, lane);
        t.b.init(t.n0, ld_bytes, wave, lane);
        t.tail_a = t.a.tail_voff(k_bytes % kRowBytes);
        t.tail_b = t.b.tail_voff(k_bytes % kRowBytes);
        t.k_rot = (slot % kNumXCD) * (k_tiles_run / kNumXCD);
        return t;
    };
    // The tiles of different XCDs (slot % 8: a property of the tile, not of the workgroup that happens to run it) start their
    // walk over K at different k-tiles and wrap around: the whole chip asking the memory side for the same columns of
    // every row at the same moment queues on the channels that hold them (8192 x 8192 x 9216: 954 -> 890 us; nothing
    // changes at K = 8192). The order of summation over K therefore depends on the tile, not on the launch.
    auto copy_pass = [&](const TileIo& t, int d, int kt_run, uint8_t* la, uint8_t* lb) {
        const int kt = kt_run + t.k_rot >= k_tiles_run ? kt_run + t.k_rot - k_tiles_run : kt_run + t.k_rot;
        const bool tail = kt == tail_tile, past = kt >= num_k_tiles;
        if (d < StA::PASSES) t.a.issue_pass_from(rsrc_a, la, kt * kRowBytes, wave, d, past ? kOutOfRange : (tail ? t.tail_a : t.a.voff));
        else t.b.issue_pass_from(rsrc_b, lb, kt * kRowBytes, wave, d - StA::PASSES, past ? kOutOfRange : (tail ? t.tail_b : t.b.voff));
    };

    // The two MFMAs that cover a 64-deep k-tile: lane group g takes chunks 2g and 2g + 1 of its row, so the first MFMA
    // contracts over chunks {0, 2, 4, 6} and the second over {1, 3, 5, 7}; both operands use the same assignment, which
    // is all the contraction needs. With chunks g and 4 + g instead (K in natural order) every ds_read_b128 takes twice
    // as long: the counters show 8 LDS cycles per instruction, half of them bank conflicts, against 4 with this order.
    const int koff[2] = {frag_offset<16>(lane, 2 * g), frag_offset<16>(lane, 2 * g + 1)};

    // One array for both stages: with a separate array per stage the compiler knows which copies feed which fragment
    // reads and guards the reads with a wait for every outstanding vector-memory operation, the output stores of the
    // previous tile included; the waits below are exact instead.
    constexpr int A_BYTES = BLOCK_M * kRowBytes, STAGE_BYTES = (BLOCK_M + LDS_ROWS_B) * kRowBytes;
    __shared__ __attribute__((aligned(1024))) uint8_t stages[2 * STAGE_BYTES];
    uint8_t* const lds_a0 = stages;
    uint8_t* const lds_b0 = stages + A_BYTES;
    uint8_t* const lds_a1 = stages + STAGE_BYTES;
    uint8_t* const lds_b1 = stages + STAGE_BYTES + A_BYTES;

    f32x4 acc[TN][TM];

    // One k-tile: STEPS = 2 * TN steps of TM MFMAs (one row of atoms, one half of K); the fragments of the next step are
    // fetched before the MFMAs of this one issue (fetching two steps ahead measured no faster).
    // The MFMAs are written as instructions whose destination is their own addend. Left to the compiler, the sums
    // wander through the register file (every MFMA writes its result somewhere new), the kernel sits at the 256-register
    // limit, spills, and pays wait states wherever a fragment read lands in registers a sum has just left: 4 % of the
    // time at 8192^3. Tied, the kernel needs 220 registers.
    // Fragments live across k-tiles: the barrier that opens k-tile t + 1 sits TAIL steps before the end of k-tile t, where
    // every fragment of k-tile t is in registers; behind it the first fragments of k-tile t + 1 are fetched and the TAIL
    // steps still held are multiplied while those fetches are under way.
    // NS slots for weight fragments, step s in slot s % NS: a divisor of STEPS, so that a step's slot is the same in every k-tile
    constexpr int TAIL = 2, NS = STEPS % 4 == 0 ? 4 : (STEPS % 5 == 0 ? 5 : (STEPS % 7 == 0 ? 7 : STEPS));
    static_assert(STEPS % NS == 0 && TAIL + 1 < NS && NUM_COPIES <= STEPS - TAIL);
    Frag nf[NS], mf[2][TM];           // weight fragments, step s in slot s % NS; activation fragments of the two K halves
    auto mma = [&](int s) {
        const int half = s / TN, i = s % TN;
#pragma unroll
        for (int j = 0; j < TM; ++j) {
            if constexpr (__is_same(Elem, __bf16))
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc[i][j]) : "v"(nf[s % NS]), "v"(mf[half][j]));
            else
                asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[i][j]) : "v"(nf[s % NS]), "v"(mf[half][j]));
        }
    };
    // What the first step of the k-tile staged in (a, b) needs.
    auto fetch_first = [&](const uint8_t* a, const uint8_t* b) {
        nf[0] = *reinterpret_cast<const Frag*>(b + wn * WTN * kRowBytes + koff[0]);
#pragma unroll
        for (int j = 0; j < TM; ++j) mf[0][j] = *reinterpret_cast<const Frag*>(a + (wm * WTM + j * 16) * kRowBytes + koff[0]);
    };
    // every copy, store and fragment read of mine is done; then: every wave's
    auto open_next = [&] {
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    // One k-tile, staged in (a_cur, b_cur), whose first fragments are in registers or on their way. `copy(s)` runs once per
    // step for the first NUM_COPIES steps and starts the copies of the k-tile that comes next, staged in (a_nxt, b_nxt).
    auto k_step = [&](const uint8_t* a_cur, const uint8_t* b_cur, const uint8_t* a_nxt, const uint8_t* b_nxt, auto&& copy) {
        const uint8_t* pa = a_cur + wm * WTM * kRowBytes;
        const uint8_t* pb = b_cur + wn * WTN * kRowBytes;
        auto fetch_n = [&](int s) { nf[s % NS] = *reinterpret_cast<const Frag*>(pb + (s % TN) * 16 * kRowBytes + koff[s / TN]); };
#pragma unroll
        for (int s = 0; s < STEPS - TAIL; ++s) {
            if (s < NUM_COPIES) copy(s);
            fetch_n(s + 1);
            if (s == STEPS - TAIL - 1) {
#pragma unroll
                for (int x = s + 2; x < STEPS; ++x) fetch_n(x);
            }
            if (s + 1 == TN) {
#pragma unroll
                for (int j = 0; j < TM; ++j) mf[1][j] = *reinterpret_cast<const Frag*>(pa + j * 16 * kRowBytes + koff[1]);
            }
            mma(s);
            __builtin_amdgcn_sched_barrier(0);        // without it the compiler hoists the reads and copies of the whole k-tile
        }
        open_next();
        fetch_first(a_nxt, b_nxt);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = STEPS - TAIL; s < STEPS; ++s) {
            mma(s);
            __builtin_amdgcn_sched_barrier(0);
        }
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
#pragma unroll
    for (int d = 0; d < NUM_COPIES; ++d) copy_pass(cur, d, 0, lds_a0, lds_b0);
    open_next();
    fetch_first(lds_a0, lds_b0);
    while (true) {
        slot = seek(slot + gridDim.x);
        const TileIo nxt = open_tile(slot);
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        int kt = 0;
        for (; kt + 2 < k_tiles_run; kt += 2) {
            k_step(lds_a0, lds_b0, lds_a1, lds_b1, [&](int s) { copy_pass(cur, s, kt + 1, lds_a1, lds_b1); });
            k_step(lds_a1, lds_b1, lds_a0, lds_b0, [&](int s) { copy_pass(cur, s, kt + 2, lds_a0, lds_b0); });
        }
        k_step(lds_a0, lds_b0, lds_a1, lds_b1, [&](int s) { copy_pass(cur, s, kt + 1, lds_a1, lds_b1); });
        // last k-tile of this tile: the copies are the first k-tile of the next tile, if there is one, and what is fetched
        // behind the barrier are its first fragments (bytes nobody uses when there is none)
        k_step(lds_a1, lds_b1, lds_a0, lds_b0, [&](int s) { if (nxt.valid) copy_pass(nxt, s, 0, lds_a0, lds_b0); });
        uint8_t* const a_last = lds_a1;
        uint8_t* const b_last = lds_b1;
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");      // the last MFMAs retire before the epilogue reads the sums

        // Epilogue: the 4 registers of atom (i, j) are n = n_slab + 16 i + 4 g + {0..3} of row m = m_slab + 16 j + col.
        // Stored straight from there a wave instruction would write 16 rows x 32 bytes; instead each wave turns its slab
        // round through the stage that was consumed last, 16 rows at a time, and stores whole row segments of 2 * WTN
        // consecutive bytes, 16 bytes per lane: 4 rows x 256 bytes per instruction for the 256-wide tile. Rows are
        // 2 * WTN + 16 bytes apart in LDS so that the 8-byte writes of 16 rows spread over the banks. The other stage is
        // receiving the next tile meanwhile.
        const int m_slab = cur.m0 + wm * WTM, n_slab = cur.n0 + wn * WTN;
        static_assert(sizeof(Elem) == 2);
        if ((n % 8) == 0) {
            constexpr int PITCH = 2 * WTN + 16;
            // lanes per row segment; rows one store instruction covers (lanes beyond the last whole row sit idle when the
            // segment length does not divide the wave); store instructions per 16 rows
            constexpr int LANES_PER_ROW = WTN / 8, ROWS_PER_STORE = kWaveSize / LANES_PER_ROW, STORES = ceil_div(16, ROWS_PER_STORE);
            static_assert((NW / 2) * 16 * PITCH <= A_BYTES && (NW / 2) * 16 * PITCH <= LDS_ROWS_B * kRowBytes);
            // every wave has read the last k-tile: they all passed the barrier inside its k_step with its fragments in registers
            uint8_t* region = (wave < NW / 2 ? a_last : b_last) + (wave % (NW / 2)) * (16 * PITCH);
            const __amdgpu_buffer_rsrc_t rsrc_c = make_out_rsrc(C + size_t(cur.m0) * n + cur.n0);
            const int r_in = lane / LANES_PER_ROW, c = lane % LANES_PER_ROW;
            const int nn = n_slab + 8 * c;
#pragma unroll
            for (int j = 0; j < TM; ++j) {
#pragma unroll
                for (int i = 0; i < TN; ++i)
                    *reinterpret_cast<decltype(pack4(acc[0][0], Elem{}))*>(region + col * PITCH + (16 * i + 4 * g) * 2) = pack4(acc[i][j], Elem{});
#pragma unroll
                for (int q = 0; q < STORES; ++q) {
                    const int row = ROWS_PER_STORE * q + r_in, mm = m_slab + 16 * j + row;
                    if (r_in < ROWS_PER_STORE && row < 16) {
                        const i32x4 v = *reinterpret_cast<const i32x4*>(region + row * PITCH + c * 16);
                        if (mm < m && nn < n)
                            buffer_store_16(v, rsrc_c, uint32_t((wm * WTM + 16 * j + row) * n + wn * WTN + 8 * c) * 2u, stream_out);
                    }
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                const int mm = m_slab + j * 16 + col;
                if (mm >= m) continue;
                Elem* row = C + size_t(mm) * n;
#pragma unroll
                for (int i = 0; i < TN; ++i) {
                    const int nn = n_slab + i * 16 + 4 * g;
                    if (nn < n) *reinterpret_cast<decltype(pack4(acc[i][j], Elem{}))*>(row + nn) = pack4(acc[i][j], Elem{});
                }
            }
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

// The 256 x 256 tile with 4 waves (one per SIMD), each with a 128 x 128 slab of 16x16x32 atoms: 256 sums per lane, pinned in
// the accumulation registers, and two thirds of the LDS fragment reads the 8-wave layout needs per k-tile (128 KB against
// 192 KB), which is what counts where the chip's power limit sets the pace. A lone wave per SIMD has nobody to hide behind:
// whatever it issues besides MFMAs has to fit the shadow of the MFMA in front of it, so
//   * every copy, fragment read and scalar update sits behind an MFMA of its own, at most one between two MFMAs;
//   * the fragments of a whole k-half (8 + 8 of them) are double-buffered in registers: a k-half is read out of LDS while
//     the k-half before it is multiplied, three reads per row of 8 MFMAs, all of them back when the k-half ends;
//   * LDS is a ring of five 32 KB units, a unit being one operand's k-tile: between the two k-halves of k-tile t every wave
//     has read all of t (its two units are free) and t + 1 has landed; the copies of t + 2 go out one per row of MFMAs
//     (a wave gets one copy instruction through per ~100 cycles, a row lasts 128), A during the first k-half of t into the
//     fifth unit, B during the second into the unit A of t has left. A copy has one k-tile (B) or two (A) to land, and the
//     wait in front of the barrier leaves the eight youngest copies in flight;
//   * the lane offsets of the copies are the same for both operands and every tile (8 registers); the tile's first row and
//     the place along K ride in the scalar offset, which the hardware adds before its bounds check.
// Persistent like the 8-wave kernel, same walk, same K rotation per XCD, same order of summation, same bits: from the last but
// one k-tile of a tile on the copies fetch the next tile; the epilogue turns the slab round through the fifth unit and its
// stores drain under the next tile. For k % 64 == 0, k >= 128, n % 8 == 0; the launcher sends everything else to the
// 8-wave kernel.
template <typename Elem, int BLOCK_N>
__device__ __forceinline__ void
dense_gemm_body_4w(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, Elem* __restrict__ C, int m, int n, int k) {
    // BLOCK_N: 256, or 160, 192, 224 (wave slabs of 80 to 112 columns, 5 to 7 rows of MFMAs per k-half; the weight unit of the
    // ring is then partly empty)
    static_assert(BLOCK_N % 32 == 0 && BLOCK_N >= 160 && BLOCK_N <= 256);
    constexpr int BLOCK_M = 256, TN = BLOCK_N / 32, TM = 8, WTN = BLOCK_N / 2, WTM = 128, UNITS = 5, UNIT_BYTES = 256 * kRowBytes;
    constexpr int PASSES_A = 8, PASSES_B = BLOCK_N / 32;         // copy instructions per wave and k-tile, 8 rows each
    using Frag = typename MfmaBF16_16x16x32::Frag;
    static_assert(sizeof(Elem) == 2 && sizeof(typename MfmaF16_16x16x32::Frag) == sizeof(Frag));
    __shared__ __attribute__((aligned(1024))) uint8_t ring[UNITS * UNIT_BYTES];

    const XcdTileScheduler<> sched(m, n, BLOCK_M, BLOCK_N, (long long)k * sizeof(Elem));
    const int num_slots = sched.grid_size();
    const int lane = get_lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
    const int wn = wave % 2, wm = wave / 2;
    const int g = lane / 16, col = lane % 16;
    const uint32_t ld_bytes = uint32_t(k) * 2;
    // Four consecutive passes of a wave's copies share one LDS base (M0) and differ in the instruction's immediate offset,
    // which the hardware adds on the LDS side and on the global side alike: the lane offsets take it back out, and the
    // descriptors start kCopyBias bytes early so that no lane offset goes below zero.
    constexpr uint32_t kCopyBias = 3 * 8 * kRowBytes;
    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(A - kCopyBias, uint32_t(m) * ld_bytes + kCopyBias);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(B - kCopyBias, uint32_t(n) * ld_bytes + kCopyBias);
    // as the 8-wave kernel: an even number of k-tiles per tile (an odd count gets one k-tile of zeros), the walk over K
    // starting at a k-tile that depends on the tile's XCD and wrapping round
    const int num_k_tiles = k / 64, k_tiles_run = (num_k_tiles + 1) & ~1;
    const uint32_t k_wrap = uint32_t(k_tiles_run) * kRowBytes;
    const int koff[2] = {frag_offset<16>(lane, 2 * g), frag_offset<16>(lane, 2 * g + 1)};
    const int a_lane = wm * WTM * kRowBytes, b_lane = wn * WTN * kRowBytes;
    const bool stream_out = size_t(m) * n * sizeof(Elem) > (size_t(32) << 20);

    // Wave w copies rows 64 w .. 64 w + 63 of the activation k-tile and rows BLOCK_N / 4 w .. of the weight k-tile, 8 rows per
    // pass. Pass j of the weights has the lane offsets of pass j of the activations when the tile is 256 wide.
    uint32_t voff[PASSES_A], voff_b[PASSES_B == PASSES_A ? 1 : PASSES_B];
    {
        const int sub = lane >> 3, slot = lane & 7;
#pragma unroll
        for (int j = 0; j < PASSES_A; ++j)     // logical chunk: slot ^ swizzle_of_row(8 (8 w + j) + sub)
            voff[j] = uint32_t(wave * 64 + j * 8 + sub) * ld_bytes + (slot ^ sub ^ (j & 1)) * kChunk + kCopyBias - (j & 3) * 8 * kRowBytes;
        if constexpr (PASSES_B != PASSES_A) {
#pragma unroll
            for (int j = 0; j < PASSES_B; ++j)
                voff_b[j] = uint32_t(wave * (BLOCK_N / 4) + j * 8 + sub) * ld_bytes + (slot ^ sub ^ ((wave * PASSES_B + j) & 1)) * kChunk +
                            kCopyBias - (j & 3) * 8 * kRowBytes;
        }
    }
    // Where the next copies fetch: the first rows of the tile they belong to (kOutOfRange: no such tile, they move zeros),
    // the byte along K, and the two put together (kOutOfRange for the k-tile of zeros).
    uint32_t base_a, base_b, kpos, at_a, at_b;
    auto aim = [&] {
        at_a = kpos < ld_bytes ? base_a + kpos : kOutOfRange;
        at_b = kpos < ld_bytes ? base_b + kpos : kOutOfRange;
    };
    auto aim_at = [&](TileCoord t, int slot) {
        base_a = t.valid ? uint32_t(t.m_idx * BLOCK_M) * ld_bytes : kOutOfRange;
        base_b = t.valid ? uint32_t(t.n_idx * BLOCK_N) * ld_bytes : kOutOfRange;
        kpos = uint32_t((slot % kNumXCD) * (k_tiles_run / kNumXCD)) * kRowBytes;
        aim();
    };
    // pass `r` of an operand's next k-tile into the ring unit at byte offset `unit`
    auto copy = [&](__amdgpu_buffer_rsrc_t rsrc, uint32_t at, uint32_t lane_off, int first_pass, int r, int unit) __attribute__((always_inline)) {
        auto* base = YAN_LDS_PTR(ring + unit + (first_pass + (r & 4)) * 8 * kRowBytes);
        switch (r & 3) {        // the immediate offset is part of the instruction
            case 0: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, base, kChunk, lane_off, at, 0 * 8 * kRowBytes, 0); break;
            case 1: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, base, kChunk, lane_off, at, 1 * 8 * kRowBytes, 0); break;
            case 2: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, base, kChunk, lane_off, at, 2 * 8 * kRowBytes, 0); break;
            default: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, base, kChunk, lane_off, at, 3 * 8 * kRowBytes, 0); break;
        }
    };
    auto copy_a = [&](int r, int unit) __attribute__((always_inline)) { copy(rsrc_a, at_a, voff[r], wave * PASSES_A, r, unit); };
    auto copy_b = [&](int r, int unit) __attribute__((always_inline)) {
        if constexpr (PASSES_B == PASSES_A) copy(rsrc_b, at_b, voff[r], wave * PASSES_B, r, unit);
        else copy(rsrc_b, at_b, voff_b[r], wave * PASSES_B, r, unit);
    };

    f32x4 acc[TN][TM];
    Frag nf[2][TN], mf[2][TM];

    // acc[i][j] (+)= weight fragment i x activation fragment j of fragment buffer KH; FIRST: the sums start here
    auto mma = [&](auto first_c, auto kh_c, int i, int j) __attribute__((always_inline)) {
        constexpr int KH = decltype(kh_c)::value;
        if constexpr (decltype(first_c)::value) {
            if constexpr (__is_same(Elem, __bf16))
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(acc[i][j]) : "v"(nf[KH][i]), "v"(mf[KH][j]));
            else
                asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(acc[i][j]) : "v"(nf[KH][i]), "v"(mf[KH][j]));
        } else {
            if constexpr (__is_same(Elem, __bf16))
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(nf[KH][i]), "v"(mf[KH][j]));
            else
                asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(nf[KH][i]), "v"(mf[KH][j]));
        }
    };
    // fragment number x of a k-half (the 8 activation fragments, then the 8 weight fragments) into buffer KH
    auto read = [&](auto kh_c, const uint8_t* pa, const uint8_t* pb, int x) __attribute__((always_inline)) {
        constexpr int KH = decltype(kh_c)::value;
        if (x < TM) mf[KH][x % TM] = *reinterpret_cast<const Frag*>(pa + (x % TM) * 16 * kRowBytes);
        else if (x < TM + TN) nf[KH][(x - TM) % TN] = *reinterpret_cast<const Frag*>(pb + ((x - TM) % TN) * 16 * kRowBytes);
    };
    // One k-half: TN rows of 8 MFMAs on fragment buffer KH; the reads of the next k-half (units ua, ub; chunk set RK) go into
    // buffer KH ^ 1, three a row; `copy(row, 0)`, `copy(row, 1)` (the narrower tiles have more activation passes than rows)
    // and `tail(row)` once per row.
    auto half_step = [&](auto kh_c, auto rk_c, auto first_c, int ua, int ub, auto&& copy, auto&& tail) __attribute__((always_inline)) {
        constexpr int KH = decltype(kh_c)::value, RK = decltype(rk_c)::value;
        using Other = std::integral_constant<int, KH ^ 1>;
        const uint8_t* pa = ring + ua + a_lane + koff[RK];
        const uint8_t* pb = ring + ub + b_lane + koff[RK];
#pragma unroll
        for (int i = 0; i < TN; ++i) {
            mma(first_c, kh_c, i, 0); copy(i, 0);
            __builtin_amdgcn_sched_barrier(0);
            mma(first_c, kh_c, i, 1); read(Other{}, pa, pb, 3 * i);
            __builtin_amdgcn_sched_barrier(0);
            mma(first_c, kh_c, i, 2); mma(first_c, kh_c, i, 3); read(Other{}, pa, pb, 3 * i + 1);
            __builtin_amdgcn_sched_barrier(0);
            mma(first_c, kh_c, i, 4); copy(i, 1);
            __builtin_amdgcn_sched_barrier(0);
            mma(first_c, kh_c, i, 5); read(Other{}, pa, pb, 3 * i + 2);
            __builtin_amdgcn_sched_barrier(0);
            mma(first_c, kh_c, i, 6); mma(first_c, kh_c, i, 7); tail(i);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    using Half0 = std::integral_constant<int, 0>;
    using Half1 = std::integral_constant<int, 1>;

    auto seek = [&](int slot) {
        while (slot < num_slots && !sched.tile_of(slot).valid) slot += gridDim.x;
        return slot;
    };
    int slot = seek(blockIdx.x);
    TileCoord cur = slot < num_slots ? sched.tile_of(slot) : TileCoord{0, 0, false};
    if (!cur.valid) return;
    aim_at(cur, slot);
    auto advance = [&] {
        kpos += kRowBytes;
        if (kpos == k_wrap) kpos = 0;
        aim();
    };
    // the first two k-tiles of the first tile into units 0 .. 3
#pragma unroll
    for (int r = 0; r < PASSES_A; ++r) copy_a(r, 0 * UNIT_BYTES);
#pragma unroll
    for (int r = 0; r < PASSES_B; ++r) copy_b(r, 1 * UNIT_BYTES);
    advance();
#pragma unroll
    for (int r = 0; r < PASSES_A; ++r) copy_a(r, 2 * UNIT_BYTES);
#pragma unroll
    for (int r = 0; r < PASSES_B; ++r) copy_b(r, 3 * UNIT_BYTES);
    advance();
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(PASSES_A + PASSES_B, kNoWaitLgkm));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    {
        const uint8_t* pa = ring + a_lane + koff[0];
        const uint8_t* pb = ring + UNIT_BYTES + b_lane + koff[0];
#pragma unroll
        for (int j = 0; j < TM; ++j) mf[0][j] = *reinterpret_cast<const Frag*>(pa + j * 16 * kRowBytes);
#pragma unroll
        for (int i = 0; i < TN; ++i) nf[0][i] = *reinterpret_cast<const Frag*>(pb + i * 16 * kRowBytes);
    }
    __builtin_amdgcn_sched_barrier(0);

    // byte offsets of the units that hold A and B of the current k-tile, of the next one, and of the fifth unit
    int oa = 0, ob = UNIT_BYTES, oa1 = 2 * UNIT_BYTES, ob1 = 3 * UNIT_BYTES, o5 = 4 * UNIT_BYTES;
    while (true) {
        const int next_slot = seek(slot + gridDim.x);
        const TileCoord nxt = next_slot < num_slots ? sched.tile_of(next_slot) : TileCoord{0, 0, false};
        auto k_tile = [&](auto first_c, int kt) __attribute__((always_inline)) {
            if (kt == k_tiles_run - 2) aim_at(nxt, next_slot);
            half_step(Half0{}, Half1{}, first_c, oa, ob,
                      [&](int r, int second) __attribute__((always_inline)) {
                          if (!second) copy_a(r, o5);
                          else if (TN + r < PASSES_A) copy_a(TN + r, o5);
                      }, [](int) {});
            // k-tile kt + 1 has landed (the 8 copies just issued may still be on their way); every wave is done reading k-tile kt
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(PASSES_A, 0));
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            // the copies move on along K and, behind the last copy of the k-tile, the units change roles: a few scalar
            // instructions a row, so that they ride under the MFMAs
            uint32_t next_b;
            const int into = oa;
            half_step(Half1{}, Half0{}, std::false_type{}, oa1, ob1,
                      [&](int r, int second) __attribute__((always_inline)) { if (!second) copy_b(r, into); },
                      [&](int r) __attribute__((always_inline)) {
                          if (r == TN - 5) { kpos += kRowBytes; if (kpos == k_wrap) kpos = 0; }
                          if (r == TN - 4) at_a = kpos < ld_bytes ? base_a + kpos : kOutOfRange;
                          if (r == TN - 3) next_b = kpos < ld_bytes ? base_b + kpos : kOutOfRange;
                          if (r == TN - 2) { const int ta = oa1; oa1 = o5; o5 = ob; ob = ob1; ob1 = oa; oa = ta; }
                          if (r == TN - 1) at_b = next_b;
                      });
        };
        k_tile(std::true_type{}, 0);
        for (int kt = 1; kt < k_tiles_run; ++kt) k_tile(std::false_type{}, kt);
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");      // the last MFMAs retire before the epilogue reads the sums

        // Epilogue: the 4 registers of atom (i, j) are n = n_slab + 16 i + 4 g + {0..3} of row m = m_slab + 16 j + col. Each wave
        // turns its slab round through the fifth unit (B of the last k-tile: every wave left it at the last barrier, the next
        // copies into it come behind the barrier below), a piece of 16 rows at a time (half the slab's width for the 256-wide
        // tile, all of it for the narrower ones) through two buffers of its own: the sums of piece u go into LDS, piece u - 1
        // comes back out as whole row segments, 16 bytes per lane, piece u - 2 is stored, so that no step waits for the LDS
        // round trip of its own piece. Rows are a segment and 16 bytes apart in LDS (the 8-byte writes of 16 rows spread over
        // the banks). Lane offsets are fixed, the piece rides in the scalar offset; rows past m fall off the end of the
        // descriptor, lanes past n or past the piece's 16 rows are sent there.
        auto epilogue = [&](auto policy_c) __attribute__((always_inline)) {
            constexpr int PIECE_COLS = BLOCK_N == 256 ? 64 : WTN, PIECES_PER_GROUP = WTN / PIECE_COLS, PIECES = TM * PIECES_PER_GROUP;
            constexpr int PITCH = 2 * PIECE_COLS + 16, PIECE_BYTES = 16 * PITCH;
            constexpr int LANES_PER_ROW = PIECE_COLS / 8, ROWS_PER_STORE = kWaveSize / LANES_PER_ROW, STORES = ceil_div(16, ROWS_PER_STORE);
            static_assert(4 * 2 * PIECE_BYTES + 8 * PITCH <= UNIT_BYTES);
            uint8_t* buffers = ring + o5 + wave * (2 * PIECE_BYTES);
            const int m0 = cur.m_idx * BLOCK_M, n0 = cur.n_idx * BLOCK_N;
            const size_t left = (size_t(m - m0) * n - n0) * sizeof(Elem);
            const __amdgpu_buffer_rsrc_t rsrc_c = make_rsrc(C + size_t(m0) * n + n0, left < kOutOfRange ? uint32_t(left) : kOutOfRange);
            const int r_in = lane / LANES_PER_ROW, c = lane % LANES_PER_ROW;    // a lane stores 16 bytes of row ROWS_PER_STORE s + r_in
            uint32_t off[PIECES_PER_GROUP];
#pragma unroll
            for (int h = 0; h < PIECES_PER_GROUP; ++h)
                off[h] = r_in < ROWS_PER_STORE && n0 + wn * WTN + PIECE_COLS * h + 8 * c < n
                             ? uint32_t((wm * WTM + r_in) * n + wn * WTN + PIECE_COLS * h + 8 * c) * 2u : kOutOfRange;
            const uint32_t row_bytes = uint32_t(n) * 2u;
            i32x4 back[2][STORES];
            auto into_lds = [&](int u) __attribute__((always_inline)) {
                const int j = u / PIECES_PER_GROUP, h = u % PIECES_PER_GROUP;
#pragma unroll
                for (int a = 0; a < PIECE_COLS / 16; ++a) {
                    // the sums come out of the accumulation registers here and nowhere earlier (left to the register
                    // allocator it moves all of them at once and spills what else is live)
                    const int i = h * (PIECE_COLS / 16) + a;
                    f32x4 sums;
                    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(sums[0]) : "a"(acc[i][j][0]));
                    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(sums[1]) : "a"(acc[i][j][1]));
                    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(sums[2]) : "a"(acc[i][j][2]));
                    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(sums[3]) : "a"(acc[i][j][3]));
                    *reinterpret_cast<decltype(pack4(sums, Elem{}))*>(buffers + (u & 1) * PIECE_BYTES + col * PITCH + (16 * a + 4 * g) * 2) = pack4(sums, Elem{});
                }
            };
            auto out_of_lds = [&](int u) __attribute__((always_inline)) {
#pragma unroll
                for (int s = 0; s < STORES; ++s)
                    back[u & 1][s] = *reinterpret_cast<const i32x4*>(buffers + (u & 1) * PIECE_BYTES + (ROWS_PER_STORE * s + r_in) * PITCH + c * 16);
            };
            auto store = [&](int u) __attribute__((always_inline)) {
                const int j = u / PIECES_PER_GROUP, h = u % PIECES_PER_GROUP;
#pragma unroll
                for (int s = 0; s < STORES; ++s) {
                    // the last store of a piece may reach past its 16 rows
                    const uint32_t lane_off = (16 % ROWS_PER_STORE == 0 || ROWS_PER_STORE * s + r_in < 16) ? off[h] : kOutOfRange;
                    __builtin_amdgcn_raw_buffer_store_b128(back[u & 1][s], rsrc_c, lane_off, (16 * j + ROWS_PER_STORE * s) * row_bytes, decltype(policy_c)::value);
                }
            };
#pragma unroll
            for (int u = 0; u < PIECES + 2; ++u) {
                if (u < PIECES) into_lds(u);
                __builtin_amdgcn_sched_barrier(0);
                if (u >= 1 && u - 1 < PIECES) out_of_lds(u - 1);
                if (u >= 2) store(u - 2);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // an output larger than the L2s together is stored with the non-temporal hint (see the 8-wave kernel)
        if (stream_out) epilogue(std::integral_constant<int, 2>{});
        else epilogue(std::integral_constant<int, 0>{});
        if (!nxt.valid) break;
        cur = nxt;
        slot = next_slot;
        // every wave is out of the fifth unit before the next copies go into it
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoWaitVm, 0));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    }
}

template <typename Elem, int BLOCK_N>
__global__ void __launch_bounds__(4 * kWaveSize)
dense_gemm_mfma_4w(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, Elem* __restrict__ C, int m, int n, int k) {
    dense_gemm_body_4w<Elem, BLOCK_N>(A, B, C, m, n, k);
}

template <typename Atom, typename Elem, int BLOCK_M, int BLOCK_N>
__global__ void __launch_bounds__(8 * kWaveSize)
dense_gemm_mfma_8w(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, Elem* __restrict__ C, int m, int n, int k) {
    dense_gemm_body_8w<Atom, Elem, BLOCK_M, BLOCK_N>(A, B, C, m, n, k);
}

// Workgroup b runs tiles b, b + gridDim.x, ...: exactly one when the launcher starts a workgroup per tile, several under
// a compute-unit cap. Between two tiles every wave must have left the epilogue of the first, which reads an LDS stage
// the second one's first copies go into.
template <typename Atom, typename Elem, int BLOCK_M, int BLOCK_N, int STAGES>
__device__ __forceinline__ void
dense_gemm_walk(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, Elem* __restrict__ C, int m, int n, int k, int num_slots) {
    // a workgroup per tile (no cap): the tile without a loop around it (up to 2 % faster than one trip round the loop below)
    if (int(gridDim.x) >= num_slots) {
        dense_gemm_body<Atom, Elem, BLOCK_M, BLOCK_N, STAGES>(A, B, C, m, n, k, int(blockIdx.x));
        return;
    }
    for (int slot = blockIdx.x; slot < num_slots; slot += gridDim.x) {
        dense_gemm_body<Atom, Elem, BLOCK_M, BLOCK_N, STAGES>(A, B, C, m, n, k, slot);
        if (slot + int(gridDim.x) < num_slots) __syncthreads();
    }
}

template <typename Atom, typename Elem, int BLOCK_M, int BLOCK_N, int STAGES>
__global__ void __launch_bounds__(4 * kWaveSize)
dense_gemm_mfma(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, Elem* __restrict__ C, int m, int n, int k, int num_slots) {
    dense_gemm_walk<Atom, Elem, BLOCK_M, BLOCK_N, STAGES>(A, B, C, m, n, k, num_slots);
}

// The ring tiles with K split SPLIT_K ways: launch slot s is part s % SPLIT_K of tile slot s / SPLIT_K.
template <typename Atom, typename Elem, int BLOCK_M, int BLOCK_N, int STAGES, int SPLIT_K>
__global__ void __launch_bounds__(4 * kWaveSize)
dense_gemm_split_k(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, Elem* __restrict__ C, int m, int n, int k,
                   float* __restrict__ partials, unsigned* __restrict__ counters) {
    dense_gemm_body<Atom, Elem, BLOCK_M, BLOCK_N, STAGES, SPLIT_K>(A, B, C, m, n, k, int(blockIdx.x), partials, counters);
}

// The fp16 flavour under the name of the reference's kernel (yan/include/gemm/cute_gemm.cuh:20), so that profiler
// filters written for it (tests/test_cute.py:35 looks for 'fp16_gemm_cute') keep finding it.
template <int BLOCK_M, int BLOCK_N, int STAGES>
__global__ void __launch_bounds__(4 * kWaveSize)
fp16_gemm_cute(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, _Float16* __restrict__ C, int m, int n, int k, int num_slots) {
    dense_gemm_walk<MfmaF16_32x32x16, _Float16, BLOCK_M, BLOCK_N, STAGES>(A, B, C, m, n, k, num_slots);
}

template <int BLOCK_M, int BLOCK_N, int STAGES, int SPLIT_K>
__global__ void __launch_bounds__(4 * kWaveSize)
fp16_gemm_cute_split_k(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, _Float16* __restrict__ C, int m, int n, int k,
                       float* __restrict__ partials, unsigned* __restrict__ counters) {
    dense_gemm_body<MfmaF16_32x32x16, _Float16, BLOCK_M, BLOCK_N, STAGES, SPLIT_K>(A, B, C, m, n, k, int(blockIdx.x), partials, counters);
}

template <int BLOCK_N>
__global__ void __launch_bounds__(4 * kWaveSize)
fp16_gemm_cute_4w(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, _Float16* __restrict__ C, int m, int n, int k) {
    dense_gemm_body_4w<_Float16, BLOCK_N>(A, B, C, m, n, k);
}

template <int BLOCK_M, int BLOCK_N>
__global__ void __launch_bounds__(8 * kWaveSize)
fp16_gemm_cute_8w(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, _Float16* __restrict__ C, int m, int n, int k) {
    dense_gemm_body_8w<MfmaF16_16x16x32, _Float16, BLOCK_M, BLOCK_N>(A, B, C, m, n, k);
}

// Arguments every dense launcher checks before touching the GPU. Returns hipSuccess or hipErrorInvalidValue.
inline hipError_t check_dense_args(int m, int n, int k, const void* a, const void* b, const void* c,
                                   int block_m, int block_n) {
    if (m < 0 || n < 0 || k <= 0 || (n % 4) != 0 || (k % 8) != 0) return hipErrorInvalidValue;
    if (!a || !b || !c) return hipErrorInvalidValue;
    // 32-bit descriptor offsets: every tile row, including the overhang of the last tile, must stay below 2 GiB
    const uint64_t m_pad = uint64_t(ceil_div(m, block_m)) * block_m, n_pad = uint64_t(ceil_div(n, block_n)) * block_n;
    if (m_pad * k * 2 >= kOutOfRange || n_pad * k * 2 >= kOutOfRange) return hipErrorInvalidValue;
    // output stores address a tile with 32-bit byte offsets from its first element: block_m rows of n elements
    if (uint64_t(block_m) * n * 2 >= kOutOfRange) return hipErrorInvalidValue;
    return hipSuccess;
}

// `num_sms`: the caller's compute-unit cap (0 = none), see capped_grid in scheduler.hpp.
// WAVES: 0 lets the launcher choose between the two kernels of the 256 x 256 tile, 8 names the 8-wave one (for comparisons).
template <typename Atom, typename Elem, int BLOCK_M, int BLOCK_N, int STAGES = DenseTileConfig<BLOCK_M, BLOCK_N>::MAX_STAGES, int WAVES = 0>
inline hipError_t launch_dense(int m, int n, int k, const void* a, const void* b, void* c, hipStream_t stream, int num_sms = 0) {
    if (m == 0 || n == 0) return hipSuccess;
    if (hipError_t e = check_dense_args(m, n, k, a, b, c, BLOCK_M, BLOCK_N); e != hipSuccess) return e;
    const XcdTileScheduler<> sched(m, n, BLOCK_M, BLOCK_N);
    const int slots = sched.grid_size();
    if constexpr (BLOCK_M == 256 && STAGES == 2) {
        // persistent: one workgroup per CU (a multiple of the 8 XCDs, so a workgroup's tiles stay on one XCD's range),
        // or as many as the caller's cap allows
        const int cus = device_cu_count() / kNumXCD * kNumXCD;
        const int grid = capped_grid(slots < cus ? slots : cus, num_sms, device_cu_count());
        // The tiles of 256 rows and 160 to 256 columns have two kernels that give the same bits: 4 waves with slabs of 128 rows
        // where its conditions hold (whole k-tiles, output rows of whole 16-byte segments) and K is long enough for it to pay
        // (256 x 256: level at k = 256, 5 to 14 % faster from k = 1024 on; the narrower tiles gain 8 to 20 %), 8 waves with
        // slabs of 64 rows otherwise.
        // (its copies address the operands 3 KB above their descriptors' start: that much less than 2 GiB per operand)
        const uint64_t m_pad = uint64_t(ceil_div(m, BLOCK_M)) * BLOCK_M, n_pad = uint64_t(ceil_div(n, BLOCK_N)) * BLOCK_N;
        const bool in_reach = (m_pad > n_pad ? m_pad : n_pad) * k * 2 + 4096 < kOutOfRange;
        if constexpr (WAVES == 0 && BLOCK_N >= 160)
        if (k % 64 == 0 && k >= 256 && n % 8 == 0 && in_reach) {
            if constexpr (__is_same(Elem, _Float16))
                hipLaunchKernelGGL((fp16_gemm_cute_4w<BLOCK_N>), dim3(grid), dim3(4 * kWaveSize), 0, stream,
                                   static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b), static_cast<Elem*>(c), m, n, k);
            else
                hipLaunchKernelGGL((dense_gemm_mfma_4w<Elem, BLOCK_N>), dim3(grid), dim3(4 * kWaveSize), 0, stream,
                                   static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b), static_cast<Elem*>(c), m, n, k);
            return hipGetLastError();
        }
        if constexpr (__is_same(Elem, _Float16))
            hipLaunchKernelGGL((fp16_gemm_cute_8w<BLOCK_M, BLOCK_N>), dim3(grid), dim3(8 * kWaveSize), 0, stream,
                               static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b), static_cast<Elem*>(c), m, n, k);
        else
            hipLaunchKernelGGL((dense_gemm_mfma_8w<MfmaBF16_16x16x32, Elem, BLOCK_M, BLOCK_N>), dim3(grid),
                               dim3(8 * kWaveSize), 0, stream, static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b),
                               static_cast<Elem*>(c), m, n, k);
    } else {
        using Cfg = DenseTileConfig<BLOCK_M, BLOCK_N>;
        const int grid = capped_grid(slots, num_sms, device_cu_count());
        if constexpr (__is_same(Elem, _Float16))
            hipLaunchKernelGGL((fp16_gemm_cute<BLOCK_M, BLOCK_N, STAGES>), dim3(grid),
                               dim3(Cfg::NUM_WAVES * kWaveSize), 0, stream, static_cast<const uint8_t*>(a),
                               static_cast<const uint8_t*>(b), static_cast<Elem*>(c), m, n, k, slots);
        else
            hipLaunchKernelGGL((dense_gemm_mfma<Atom, Elem, BLOCK_M, BLOCK_N, STAGES>), dim3(grid),
                               dim3(Cfg::NUM_WAVES * kWaveSize), 0, stream, static_cast<const uint8_t*>(a),
                               static_cast<const uint8_t*>(b), static_cast<Elem*>(c), m, n, k, slots);
    }
    return hipGetLastError();
}

// K split SPLIT_K ways over as many workgroups per tile (ring tiles). `workspace`: device memory of at least
// kSplitKCounterBytes + tile slots * SPLIT_K * BLOCK_M * BLOCK_N * 4 bytes: counters that are zero before the first launch and
// after every launch, then the partial sums. Launches that share a workspace must not overlap (see fp8_gemm.hpp).
template <typename Atom, typename Elem, int BLOCK_M, int BLOCK_N, int SPLIT_K, int STAGES = DenseTileConfig<BLOCK_M, BLOCK_N>::MAX_STAGES>
inline hipError_t launch_dense_split_k(int m, int n, int k, const void* a, const void* b, void* c, hipStream_t stream,
                                       void* workspace, size_t workspace_bytes) {
    static_assert(SPLIT_K > 1 && !(BLOCK_M == 256 && STAGES == 2));
    if (m == 0 || n == 0) return hipSuccess;
    if (hipError_t e = check_dense_args(m, n, k, a, b, c, BLOCK_M, BLOCK_N); e != hipSuccess) return e;
    if (!workspace) return hipErrorInvalidValue;
    using Cfg = DenseTileConfig<BLOCK_M, BLOCK_N>;
    const XcdTileScheduler<> sched(m, n, BLOCK_M, BLOCK_N);
    const size_t slots = size_t(sched.grid_size());
    if (slots * Cfg::NUM_WAVES * 4 > kSplitKCounterBytes) return hipErrorInvalidValue;
    if (workspace_bytes < kSplitKCounterBytes + slots * SPLIT_K * BLOCK_M * BLOCK_N * 4) return hipErrorInvalidValue;
    unsigned* counters = static_cast<unsigned*>(workspace);
    float* partials = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + kSplitKCounterBytes);
    if constexpr (__is_same(Elem, _Float16))
        hipLaunchKernelGGL((fp16_gemm_cute_split_k<BLOCK_M, BLOCK_N, STAGES, SPLIT_K>), dim3(int(slots) * SPLIT_K),
                           dim3(Cfg::NUM_WAVES * kWaveSize), 0, stream, static_cast<const uint8_t*>(a),
                           static_cast<const uint8_t*>(b), static_cast<Elem*>(c), m, n, k, partials, counters);
    else
        hipLaunchKernelGGL((dense_gemm_split_k<Atom, Elem, BLOCK_M, BLOCK_N, STAGES, SPLIT_K>), dim3(int(slots) * SPLIT_K),
                           dim3(Cfg::NUM_WAVES * kWaveSize), 0, stream, static_cast<const uint8_t*>(a),
                           static_cast<const uint8_t*>(b), static_cast<Elem*>(c), m, n, k, partials, counters);
    return hipGetLastError();
}

} // namespace yan

// bf16 in, fp32 accumulate, bf16 out. NUM_STAGES is the number of LDS stages (2 .. DenseTileConfig::MAX_STAGES; two
// 256x256x64 stages are 128 KB of the 160 KB, smaller tiles can hold a deeper ring).
template <int BLOCK_M, int BLOCK_N, int NUM_STAGES, int WAVES = 0>
inline hipError_t gemm_tn(int m, int n, int k, const __hip_bfloat16* A, const __hip_bfloat16* B, __hip_bfloat16* C,
                          hipStream_t stream, int num_sms = 0) {
    // BLOCK_N == 16 names the weight-streaming kernel for up to BLOCK_M activation rows (bf16_gemm_skinny.hpp)
    if constexpr (BLOCK_N == 16) return yan::launch_dense_skinny<yan::MfmaBF16_16x16x32, __bf16, BLOCK_M / 16, 8>(m, n, k, A, B, C, stream);
    else return yan::launch_dense<yan::MfmaBF16_32x32x16, __bf16, BLOCK_M, BLOCK_N, NUM_STAGES, WAVES>(m, n, k, A, B, C, stream, num_sms);
}

// fp16 in, fp32 accumulate, fp16 out.
template <int BLOCK_M, int BLOCK_N, int NUM_STAGES, int SPLIT_K>
inline hipError_t gemm_tn_split_k(int m, int n, int k, const __hip_bfloat16* A, const __hip_bfloat16* B, __hip_bfloat16* C,
                                  hipStream_t stream, void* workspace, size_t workspace_bytes) {
    return yan::launch_dense_split_k<yan::MfmaBF16_32x32x16, __bf16, BLOCK_M, BLOCK_N, SPLIT_K, NUM_STAGES>(m, n, k, A, B, C, stream, workspace, workspace_bytes);
}

template <int BLOCK_M, int BLOCK_N, int NUM_STAGES, int SPLIT_K>
inline hipError_t gemm_tn_split_k(int m, int n, int k, const __half* A, const __half* B, __half* C, hipStream_t stream,
                                  void* workspace, size_t workspace_bytes) {
    return yan::launch_dense_split_k<yan::MfmaF16_32x32x16, _Float16, BLOCK_M, BLOCK_N, SPLIT_K, NUM_STAGES>(m, n, k, A, B, C, stream, workspace, workspace_bytes);
}

template <int BLOCK_M, int BLOCK_N, int NUM_STAGES, int WAVES = 0>
inline hipError_t gemm_tn(int m, int n, int k, const __half* A, const __half* B, __half* C, hipStream_t stream, int num_sms = 0) {
    if constexpr (BLOCK_N == 16) return yan::launch_dense_skinny<yan::MfmaF16_16x16x32, _Float16, BLOCK_M / 16, 8>(m, n, k, A, B, C, stream);
    else return yan::launch_dense<yan::MfmaF16_32x32x16, _Float16, BLOCK_M, BLOCK_N, NUM_STAGES, WAVES>(m, n, k, A, B, C, stream, num_sms);
}
