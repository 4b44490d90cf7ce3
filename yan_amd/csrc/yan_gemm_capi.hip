// Ahead-of-time C-ABI library over the JIT's kernel headers: every tile variant instantiated once, sizes at run time.
// Declarations and contracts: include/yan_gemm.h.
#include "../../include/yan_gemm.h"

#include "gemm/bf16_gemm.hpp"
#include "gemm/fp8_gemm.hpp"
#include "gemm/fp8_gemm_skinny.hpp"
#include "gemm/bf16_gemm_skinny.hpp"
#include "gemm/fp8_cast.hpp"
#include "gemm/simple_gemm.hpp"

#include <mutex>

// Scratch of the entry point that allocates nothing (yan_gemm_fp8_fp8_bf16_nt_static): the split-K workspace as a device
// array. Every GPU the library runs on holds its own copy, zero when the module is loaded, until the process ends; host
// code reaches a GPU's copy through the address hipGetSymbolAddress returns with that GPU current, never through the name.
static __device__ __align__(256) unsigned char scratch[yan::kSplitKWorkspaceBytes];

namespace {

struct TileCost { int bm, bn; double per_area; };

// Same tables and cost model as yan_amd/jit_kernels/heuristics.py (a CPU test keeps the two in step).
constexpr TileCost kDenseTiles[] = {{256, 256, 1.00}, {256, 224, 1.03}, {256, 192, 1.05}, {256, 160, 1.085}, {256, 128, 1.42}, {128, 256, 1.40},
                                    {128, 192, 1.43}, {128, 128, 1.51}, {64, 192, 1.96}, {64, 128, 2.0}, {64, 64, 2.78}};
constexpr TileCost kFp8Tiles[]   = {{256, 256, 1.00}, {256, 192, 1.12}, {256, 160, 1.28}, {256, 128, 1.34}, {128, 256, 1.34}, {128, 128, 1.5},
                                    {64, 128, 2.3}, {64, 64, 3.55}, {64, 32, 4.8}, {32, 32, 7.0}};

template <int COUNT>
void pick(const TileCost (&tiles)[COUNT], int m, int n, int num_cus, int* bm, int* bn) {
    double best = -1;
    for (const TileCost& t : tiles) {
        const long long count  = (long long)((m + t.bm - 1) / t.bm) * ((n + t.bn - 1) / t.bn);
        const long long rounds = (count + num_cus - 1) / num_cus;
        const double cost = double(rounds) * t.bm * t.bn * t.per_area;
        // ties go to the earlier entry of the (cost, tile) ordering the Python side sorts by
        if (best < 0 || cost < best || (cost == best && (t.bm < *bm || (t.bm == *bm && t.bn < *bn)))) { best = cost; *bm = t.bm; *bn = t.bn; }
    }
}

// Tile of a grouped FP8 GEMM (get_best_grouped_fp8_config in heuristics.py): tiles 64, 128 or 256 wide; with a non-zero
// `m_alignment` BLOCK_M divides it, or is twice it when the `groups_in_m` groups average 1024 rows or more; the tile
// count is multiplied by `groups`.
void pick_grouped(int m, int n, int num_cus, int groups, int m_alignment, int groups_in_m, int* bm, int* bn) {
    double best = -1;
    if (m < 1) m = 1;
    for (const TileCost& t : kFp8Tiles) {
        const bool fits = m_alignment == 0 || m_alignment % t.bm == 0 ||
                          (t.bm == 2 * m_alignment && (long long)m >= 1024ll * groups_in_m);
        if ((t.bn != 64 && t.bn != 128 && t.bn != 256) || !fits) continue;
        const long long count  = (long long)((m + t.bm - 1) / t.bm) * ((n + t.bn - 1) / t.bn) * groups;
        const long long rounds = (count + num_cus - 1) / num_cus;
        const double cost = double(rounds) * t.bm * t.bn * t.per_area;
        if (best < 0 || cost < best || (cost == best && (t.bm < *bm || (t.bm == *bm && t.bn < *bn)))) { best = cost; *bm = t.bm; *bn = t.bn; }
    }
}

// Whether a contiguous grouped GEMM runs the kernel that decides on the device what its 256-row tiles do about group boundaries
// (get_contiguous_rows_on_device in heuristics.py): groups of 256 to 2047 rows on average that get 256 x 256 tiles when every
// tile height is allowed.
bool rows_on_device(int m, int n, int num_cus, int groups_in_m) {
    if (groups_in_m <= 0 || (long long)m < 256ll * groups_in_m || (long long)m >= 2048ll * groups_in_m) return false;
    // the same table with every tile height allowed
    double best = -1;
    int tm = 0, tn = 0;
    for (const TileCost& t : kFp8Tiles) {
        if ((t.bn != 64 && t.bn != 128 && t.bn != 256) || (t.bm != 64 && t.bm != 128 && t.bm != 256)) continue;
        const long long count  = (long long)((m + t.bm - 1) / t.bm) * ((n + t.bn - 1) / t.bn);
        const long long rounds = (count + num_cus - 1) / num_cus;
        const double cost = double(rounds) * t.bm * t.bn * t.per_area;
        if (best < 0 || cost < best || (cost == best && (t.bm < tm || (t.bm == tm && t.bn < tn)))) { best = cost; tm = t.bm; tn = t.bn; }
    }
    return tm == 256 && tn == 256;
}

// Activation atoms of the weight-streaming kernel, or 0 for the tiled kernel (get_skinny_fp8_config in heuristics.py).
int skinny_atoms(int m, int n, int num_cus) {
    return (m > 0 && m <= 16 && n >= 16 && n <= 16 * num_cus) ? 1 : 0;
}

// Split-K plan of the plain FP8 GEMM (get_split_k_fp8_config in heuristics.py): false when K is not split.
struct SplitKTile { int bm, bn; double us_per_k_tile, unsplit_us_per_k_tile; };
constexpr SplitKTile kSplitKTiles[] = {{32, 32, 0.133, 0.117}, {64, 32, 0.192, 0.169}, {64, 64, 0.296, 0.275}, {64, 128, 0.395, 0.375},
                                       {128, 128, 0.51, 0.497}};
constexpr int kSplitKFactors[] = {2, 3, 4};

bool pick_split_k(int m, int n, int k, int num_cus, int* bm, int* bn, int* split_k) {
    if (m <= 0 || n <= 0 || k <= 0) return false;
    const int k_tiles = k / 128;
    int ubm = 0, ubn = 0;
    pick(kFp8Tiles, m, n, num_cus, &ubm, &ubn);
    double unsplit_us = -1;
    for (const SplitKTile& t : kSplitKTiles)
        if (t.bm == ubm && t.bn == ubn) unsplit_us = t.unsplit_us_per_k_tile;
    if (unsplit_us < 0 || (long long)((m + ubm - 1) / ubm) * ((n + ubn - 1) / ubn) > num_cus) return false;
    const double floor = double((long long)n * k) / 6.0e6;
    const double unsplit_time = k_tiles * unsplit_us;
    const double base = unsplit_time > floor ? unsplit_time : floor;
    double best = -1;
    for (const SplitKTile& t : kSplitKTiles) {
        if (t.bm > 32 && t.bm >= 2 * m) continue;
        const long long tiles = (long long)((m + t.bm - 1) / t.bm) * ((n + t.bn - 1) / t.bn);
        for (const int s : kSplitKFactors) {
            const int per_part = (k_tiles + s - 1) / s;
            if ((tiles + 7) / 8 * 8 * s > (num_cus < 256 ? num_cus : 256) || per_part < (s == 2 ? 24 : 14)) continue;
            const double loop = per_part * t.us_per_k_tile + 0.5 + double(s * t.bm * t.bn * 4) / 1024 * 0.0125;
            const double time = loop > floor ? loop : floor;
            if (best < 0 || time < best) { best = time; *bm = t.bm; *bn = t.bn; *split_k = s; }
        }
    }
    return best >= 0 && base - best >= 0.10 * (base + 3.5);
}

// Split-K plan of the dense 16-bit GEMM (get_split_k_dense_config in heuristics.py): false when K is not split.
struct DenseSplitKTile { int bm, bn; double us_per_k_tile, extra_us; };      // extra < 0: not a tile plans use
constexpr DenseSplitKTile kDenseSplitKTiles[] = {{64, 64, 0.248, 0.0}, {64, 128, 0.378, 1.0}, {128, 128, 0.51, 2.5}, {64, 192, 0.60, -1},
                                                 {128, 192, 0.80, -1}, {128, 256, 0.94, -1}, {256, 128, 0.94, -1}};
constexpr int kDenseSplitKFactors[] = {2, 3, 4, 6, 8};       // six and eight parts on 64 x 64 tiles only
int dense_skinny_atoms(int m, int n, int k, int num_cus);

bool pick_dense_split_k(int m, int n, int k, int num_cus, int* bm, int* bn, int* split_k) {
    if (m <= 0 || n <= 0 || k <= 0 || ((m < 8 || (m <= 16 && k > 8192)) && dense_skinny_atoms(m, n, k, num_cus))) return false;
    const int k_tiles = (k + 63) / 64;
    int ubm = 0, ubn = 0;
    pick(kDenseTiles, m, n, num_cus, &ubm, &ubn);
    double unsplit_us = -1;
    for (const DenseSplitKTile& t : kDenseSplitKTiles)
        if (t.bm == ubm && t.bn == ubn) unsplit_us = t.us_per_k_tile;
    if (unsplit_us < 0 || (long long)((m + ubm - 1) / ubm) * ((n + ubn - 1) / ubn) > num_cus) return false;
    const double floor = double((long long)n * k * 2) / 6.0e6;
    const double unsplit_time = k_tiles * unsplit_us;
    const double base = unsplit_time > floor ? unsplit_time : floor;
    double best = -1;
    for (const DenseSplitKTile& t : kDenseSplitKTiles) {
        if (t.extra_us < 0 || (t.bm > 64 && t.bm >= 2 * m)) continue;
        const long long tiles = (long long)((m + t.bm - 1) / t.bm) * ((n + t.bn - 1) / t.bn);
        for (const int s : kDenseSplitKFactors) {
            if (s > 4 && !(t.bm == 64 && t.bn == 64)) continue;
            const int per_part = (k_tiles + s - 1) / s;
            if ((tiles + 7) / 8 * 8 * s > (num_cus < 256 ? num_cus : 256) || per_part < 16) continue;
            const double loop = per_part * t.us_per_k_tile + 0.5 + double(s * t.bm * t.bn * 4) / 1024 * 0.0125 + t.extra_us;
            const double time = loop > floor ? loop : floor;
            if (best < 0 || time < best) { best = time; *bm = t.bm; *bn = t.bn; *split_k = s; }
        }
    }
    return best >= 0 && base - best >= 0.11 * (base + 3.5);
}

int device_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    return cus;
}

// Activation atoms of the weight-streaming dense kernel, or 0 for the tiled kernels (get_skinny_dense_config in heuristics.py).
int dense_skinny_atoms(int m, int n, int k, int num_cus) {
    if (n < 16 || n > 16 * num_cus || (n % 4) != 0 || k <= 0 || (k % 64) != 0) return 0;
    if (m > 0 && m <= 16) return 1;
    if (m > 16 && m <= 32 && k >= 2048) return 2;
    return 0;
}

// With a workspace, problems the split-K plan covers run split (a workspace too small for the plan is an error); without
// one, and for every other problem, a workgroup per tile.
template <typename Atom, typename SkinnyAtom, typename Elem>
int dense(int m, int n, int k, const void* a, const void* b, void* c, void* stream, void* workspace = nullptr, size_t workspace_bytes = 0) {
    if (m == 0 || n == 0) return 0;
    if (m < 0 || n < 0) return int(hipErrorInvalidValue);
    hipStream_t s = static_cast<hipStream_t>(stream);
    int bm = 0, bn = 0, split_k = 1;
    // a split-K plan goes before the weight-streaming kernels (pick_dense_split_k makes none where the one-atom kernel is the
    // faster: below 8 rows, and up to 16 rows on K beyond 8192)
    if (workspace && pick_dense_split_k(m, n, k, device_cus(), &bm, &bn, &split_k)) {
#define YAN_DENSE_SPLIT_K_CASE(BM, BN, S) \
    if (bm == BM && bn == BN && split_k == S) return int(yan::launch_dense_split_k<Atom, Elem, BM, BN, S>(m, n, k, a, b, c, s, workspace, workspace_bytes));
#define YAN_DENSE_SPLIT_K_TILE(BM, BN) YAN_DENSE_SPLIT_K_CASE(BM, BN, 2) YAN_DENSE_SPLIT_K_CASE(BM, BN, 3) YAN_DENSE_SPLIT_K_CASE(BM, BN, 4)
        YAN_DENSE_SPLIT_K_TILE(64, 64) YAN_DENSE_SPLIT_K_TILE(64, 128) YAN_DENSE_SPLIT_K_TILE(128, 128)
        YAN_DENSE_SPLIT_K_CASE(64, 64, 6) YAN_DENSE_SPLIT_K_CASE(64, 64, 8)
#undef YAN_DENSE_SPLIT_K_TILE
#undef YAN_DENSE_SPLIT_K_CASE
        return int(hipErrorInvalidValue);
    }
    if (const int atoms = dense_skinny_atoms(m, n, k, device_cus())) {
        if (atoms == 1) return int(yan::launch_dense_skinny<SkinnyAtom, Elem, 1, 8>(m, n, k, a, b, c, s));
        return int(yan::launch_dense_skinny<SkinnyAtom, Elem, 2, 8>(m, n, k, a, b, c, s));
    }
    pick(kDenseTiles, m, n, device_cus(), &bm, &bn);
#define YAN_DENSE_CASE(BM, BN) if (bm == BM && bn == BN) return int(yan::launch_dense<Atom, Elem, BM, BN>(m, n, k, a, b, c, s));
#define YAN_DENSE_CASE_8W(BM, BN) if (bm == BM && bn == BN) return int(yan::launch_dense<Atom, Elem, BM, BN, 2>(m, n, k, a, b, c, s));
    YAN_DENSE_CASE_8W(256, 256) YAN_DENSE_CASE_8W(256, 224) YAN_DENSE_CASE_8W(256, 192) YAN_DENSE_CASE_8W(256, 160)
    YAN_DENSE_CASE(256, 128) YAN_DENSE_CASE(128, 256) YAN_DENSE_CASE(128, 192) YAN_DENSE_CASE(128, 128) YAN_DENSE_CASE(64, 192)
    YAN_DENSE_CASE(64, 128) YAN_DENSE_CASE(64, 64)
#undef YAN_DENSE_CASE
#undef YAN_DENSE_CASE_8W
    return int(hipErrorInvalidValue);
}

void* static_scratch() {
    constexpr int kMaxDevices = 64;
    static std::mutex guard;
    static void* address[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(guard);
    if (!address[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
        address[dev] = ptr;
    }
    return address[dev];
}

// The plain FP8 GEMM. With a workspace, problems the split-K plan covers run split (a workspace too small for the plan is
// an error); without one, and for every other problem, a workgroup per tile as before.
int fp8_plain(const void* lhs, const float* lhs_scales, long long lhs_scales_stride_m, long long lhs_scales_stride_k,
              const void* rhs, const float* rhs_scales, void* out, int m, int n, int k, void* stream, int num_sms,
              void* workspace, size_t workspace_bytes) {
    if (m == 0 || n == 0) return 0;
    if (m < 0 || n < 0 || k <= 0) return int(hipErrorInvalidValue);
    // the kernel addresses the scale tensor with 32-bit byte offsets
    const long long last = (long long)(m - 1) * lhs_scales_stride_m + (long long)(k / 128 - 1) * lhs_scales_stride_k;
    if (lhs_scales_stride_m < 0 || lhs_scales_stride_k < 0 || last >= (1ll << 28)) return int(hipErrorInvalidValue);
    const int cus = (num_sms > 0 && num_sms < device_cus()) ? num_sms : device_cus();
    hipStream_t s = static_cast<hipStream_t>(stream);
    __hip_bfloat16* o = static_cast<__hip_bfloat16*>(out);
    int bm = 0, bn = 0, split_k = 1;
    // a split-K plan goes before the weight-streaming kernel
    if (workspace && pick_split_k(m, n, k, cus, &bm, &bn, &split_k)) {
#define YAN_SPLIT_K_CASE(BM, BN, S)                                                                                  \
    if (bm == BM && bn == BN && split_k == S)                                                                        \
        return int(yan::Gemm<0, 0, BM, BN, 128, 1, yan::Fp8TileConfig<BM, BN>::MAX_RING_STAGES, 1, yan::GemmType::Normal>::run_split_k<S>( \
            o, lhs, lhs_scales, int(lhs_scales_stride_m), int(lhs_scales_stride_k), rhs, rhs_scales, m, n, k, s, workspace, workspace_bytes));
#define YAN_SPLIT_K_TILE(BM, BN) YAN_SPLIT_K_CASE(BM, BN, 2) YAN_SPLIT_K_CASE(BM, BN, 3) YAN_SPLIT_K_CASE(BM, BN, 4)
        YAN_SPLIT_K_TILE(32, 32) YAN_SPLIT_K_TILE(64, 32) YAN_SPLIT_K_TILE(64, 64) YAN_SPLIT_K_TILE(64, 128) YAN_SPLIT_K_TILE(128, 128)
#undef YAN_SPLIT_K_TILE
#undef YAN_SPLIT_K_CASE
        return int(hipErrorInvalidValue);
    }
    if (skinny_atoms(m, n, cus))
        return int(yan::launch_fp8_skinny<0, 0, 1, 8>(o, lhs, lhs_scales, int(lhs_scales_stride_m), int(lhs_scales_stride_k), rhs,
                                                      rhs_scales, m, n, k, s));
    pick(kFp8Tiles, m, n, cus, &bm, &bn);
#define YAN_FP8_CASE(BM, BN)                                                                                         \
    if (bm == BM && bn == BN)                                                                                        \
        return int(yan::Gemm<0, 0, BM, BN, 128, 1, yan::Fp8TileConfig<BM, BN>::MAX_RING_STAGES, 1, yan::GemmType::Normal>::run_sized(                          \
            o, lhs, lhs_scales, int(lhs_scales_stride_m), int(lhs_scales_stride_k), rhs, rhs_scales, m, n, k, s, num_sms, 0));
    YAN_FP8_CASE(256, 256) YAN_FP8_CASE(256, 192) YAN_FP8_CASE(256, 160) YAN_FP8_CASE(256, 128) YAN_FP8_CASE(128, 256) YAN_FP8_CASE(128, 128) YAN_FP8_CASE(64, 128) YAN_FP8_CASE(64, 64)
    YAN_FP8_CASE(64, 32) YAN_FP8_CASE(32, 32)
#undef YAN_FP8_CASE
    return int(hipErrorInvalidValue);
}

} // namespace

extern "C" {

int yan_gemm_bf16_tn(int m, int n, int k, const void* a, const void* b, void* c, void* stream) {
    return dense<yan::MfmaBF16_32x32x16, yan::MfmaBF16_16x16x32, __bf16>(m, n, k, a, b, c, stream);
}

int yan_gemm_fp16_tn(int m, int n, int k, const void* a, const void* b, void* c, void* stream) {
    return dense<yan::MfmaF16_32x32x16, yan::MfmaF16_16x16x32, _Float16>(m, n, k, a, b, c, stream);
}

int yan_gemm_bf16_tn_split_k(int m, int n, int k, const void* a, const void* b, void* c, void* stream, void* workspace,
                             long long workspace_bytes) {
    if (!workspace || workspace_bytes < 0) return int(hipErrorInvalidValue);
    return dense<yan::MfmaBF16_32x32x16, yan::MfmaBF16_16x16x32, __bf16>(m, n, k, a, b, c, stream, workspace, size_t(workspace_bytes));
}

int yan_gemm_fp16_tn_split_k(int m, int n, int k, const void* a, const void* b, void* c, void* stream, void* workspace,
                             long long workspace_bytes) {
    if (!workspace || workspace_bytes < 0) return int(hipErrorInvalidValue);
    return dense<yan::MfmaF16_32x32x16, yan::MfmaF16_16x16x32, _Float16>(m, n, k, a, b, c, stream, workspace, size_t(workspace_bytes));
}

int yan_gemm_float_nt(int m, int n, int k, float alpha, const float* a, int lda, const float* b, int ldb, float beta,
                      float* c, int ldc, void* stream) {
    return int(gemm_nt(m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, static_cast<hipStream_t>(stream), device_cus()));
}

int yan_gemm_fp8_fp8_bf16_nt(const void* lhs, const float* lhs_scales, long long lhs_scales_stride_m,
                             long long lhs_scales_stride_k, const void* rhs, const float* rhs_scales, void* out,
                             int m, int n, int k, void* stream, int num_sms) {
    return fp8_plain(lhs, lhs_scales, lhs_scales_stride_m, lhs_scales_stride_k, rhs, rhs_scales, out, m, n, k, stream, num_sms,
                     nullptr, 0);
}

long long yan_gemm_split_k_workspace_bytes(void) { return (long long)yan::kSplitKWorkspaceBytes; }
long long yan_gemm_split_k_counter_bytes(void) { return (long long)yan::kSplitKCounterBytes; }

int yan_gemm_fp8_fp8_bf16_nt_split_k(const void* lhs, const float* lhs_scales, long long lhs_scales_stride_m,
                                     long long lhs_scales_stride_k, const void* rhs, const float* rhs_scales, void* out,
                                     int m, int n, int k, void* stream, int num_sms, void* workspace, long long workspace_bytes) {
    if (!workspace || workspace_bytes < 0) return int(hipErrorInvalidValue);
    return fp8_plain(lhs, lhs_scales, lhs_scales_stride_m, lhs_scales_stride_k, rhs, rhs_scales, out, m, n, k, stream, num_sms,
                     workspace, size_t(workspace_bytes));
}

// Same as yan_gemm_fp8_fp8_bf16_nt_split_k with the device array `scratch` for a workspace: no allocation anywhere on the
// way. Calls on one GPU share that GPU's array: they must not overlap on the device.
int yan_gemm_fp8_fp8_bf16_nt_static(const void* lhs, const float* lhs_scales, long long lhs_scales_stride_m,
                                    long long lhs_scales_stride_k, const void* rhs, const float* rhs_scales, void* out,
                                    int m, int n, int k, void* stream, int num_sms) {
    void* workspace = static_scratch();
    if (!workspace) return int(hipErrorInvalidValue);
    return fp8_plain(lhs, lhs_scales, lhs_scales_stride_m, lhs_scales_stride_k, rhs, rhs_scales, out, m, n, k, stream, num_sms,
                     workspace, yan::kSplitKWorkspaceBytes);
}

// Arrival counters of a split-K workspace (the library's own array when `workspace` is null) back to zero, on `stream`.
int yan_gemm_split_k_reset(void* workspace, void* stream) {
    if (!workspace) workspace = static_scratch();
    return int(yan::launch_split_k_reset(workspace, yan::kSplitKCounterBytes, static_cast<hipStream_t>(stream)));
}

int yan_m_grouped_gemm_fp8_fp8_bf16_nt_contiguous(const void* lhs, const float* lhs_scales, long long lhs_scales_stride_m,
                                                  long long lhs_scales_stride_k, const void* rhs, const float* rhs_scales,
                                                  void* out, const int* m_indices, int num_groups, int m, int n, int k,
                                                  void* stream, int num_sms) {
    if (m == 0 || n == 0) return 0;
    if (m < 0 || n < 0 || k <= 0 || num_groups <= 0 || (m % 128) != 0) return int(hipErrorInvalidValue);
    const long long last = (long long)(m - 1) * lhs_scales_stride_m + (long long)(k / 128 - 1) * lhs_scales_stride_k;
    if (lhs_scales_stride_m < 0 || lhs_scales_stride_k < 0 || last >= (1ll << 28)) return int(hipErrorInvalidValue);
    const int cus = (num_sms > 0 && num_sms < device_cus()) ? num_sms : device_cus();
    if (rows_on_device(m, n, cus, num_groups))
        return int(yan::Gemm<0, 0, 256, 256, 128, 1, 2, 1, yan::GemmType::GroupedContiguous>::run_grouped_rows_on_device(
            static_cast<__hip_bfloat16*>(out), lhs, lhs_scales, int(lhs_scales_stride_m), int(lhs_scales_stride_k), rhs, rhs_scales, m_indices,
            num_groups, m, n, k, static_cast<hipStream_t>(stream), num_sms));
    int bm = 0, bn = 0;
    pick_grouped(m, n, cus, 1, 128, num_groups, &bm, &bn);
#define YAN_GROUPED_CASE(BM, BN)                                                                                     \
    if (bm == BM && bn == BN)                                                                                        \
        return int(yan::Gemm<0, 0, BM, BN, 128, 1, yan::Fp8TileConfig<BM, BN>::MAX_RING_STAGES, 1, yan::GemmType::GroupedContiguous>::run_grouped(             \
            static_cast<__hip_bfloat16*>(out), lhs, lhs_scales, int(lhs_scales_stride_m), int(lhs_scales_stride_k), 0, rhs, \
            rhs_scales, m_indices, num_groups, m, n, k, static_cast<hipStream_t>(stream), num_sms));
    YAN_GROUPED_CASE(256, 256) YAN_GROUPED_CASE(256, 128) YAN_GROUPED_CASE(128, 256) YAN_GROUPED_CASE(128, 128)
    YAN_GROUPED_CASE(64, 128) YAN_GROUPED_CASE(64, 64)
#undef YAN_GROUPED_CASE
    return int(hipErrorInvalidValue);
}

int yan_m_grouped_gemm_fp8_fp8_bf16_nt_masked(const void* lhs, const float* lhs_scales, long long lhs_scales_stride_g,
                                              long long lhs_scales_stride_m, long long lhs_scales_stride_k, const void* rhs,
                                              const float* rhs_scales, void* out, const int* masked_m, int num_groups,
                                              int m_max, int expected_m, int n, int k, void* stream, int num_sms) {
    if (m_max == 0 || n == 0 || num_groups == 0) return 0;
    if (m_max < 0 || n < 0 || k <= 0 || num_groups < 0 || expected_m <= 0) return int(hipErrorInvalidValue);
    const long long last = (long long)(m_max - 1) * lhs_scales_stride_m + (long long)(k / 128 - 1) * lhs_scales_stride_k;
    if (lhs_scales_stride_m < 0 || lhs_scales_stride_k < 0 || lhs_scales_stride_g < 0 || last >= (1ll << 28) ||
        lhs_scales_stride_g >= (1ll << 31)) return int(hipErrorInvalidValue);
    const int cus = (num_sms > 0 && num_sms < device_cus()) ? num_sms : device_cus();
    int bm = 0, bn = 0;
    pick_grouped(expected_m < m_max ? expected_m : m_max, n, cus, num_groups, 0, 1, &bm, &bn);
#define YAN_GROUPED_CASE(BM, BN)                                                                                     \
    if (bm == BM && bn == BN)                                                                                        \
        return int(yan::Gemm<0, 0, BM, BN, 128, 1, yan::Fp8TileConfig<BM, BN>::MAX_RING_STAGES, 1, yan::GemmType::GroupedMasked>::run_grouped(                 \
            static_cast<__hip_bfloat16*>(out), lhs, lhs_scales, int(lhs_scales_stride_m), int(lhs_scales_stride_k),  \
            int(lhs_scales_stride_g), rhs, rhs_scales, masked_m, num_groups, m_max, n, k, static_cast<hipStream_t>(stream), num_sms, \
            expected_m));
    YAN_GROUPED_CASE(256, 256) YAN_GROUPED_CASE(256, 128) YAN_GROUPED_CASE(128, 256) YAN_GROUPED_CASE(128, 128)
    YAN_GROUPED_CASE(64, 128) YAN_GROUPED_CASE(64, 64)
#undef YAN_GROUPED_CASE
    return int(hipErrorInvalidValue);
}

int yan_per_token_cast_to_fp8(const void* x, int x_is_fp32, void* q, float* scales, long long scales_stride_m,
                              long long scales_stride_k, int m, int k, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (x_is_fp32) return int(yan::launch_per_token_cast(static_cast<const float*>(x), q, scales, scales_stride_m, scales_stride_k, m, k, s));
    return int(yan::launch_per_token_cast(static_cast<const __bf16*>(x), q, scales, scales_stride_m, scales_stride_k, m, k, s));
}

int yan_per_block_cast_to_fp8(const void* w, int w_is_fp32, void* q, float* scales, int n, int k, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (w_is_fp32) return int(yan::launch_per_block_cast(static_cast<const float*>(w), q, scales, n, k, s));
    return int(yan::launch_per_block_cast(static_cast<const __bf16*>(w), q, scales, n, k, s));
}

int yan_gemm_select_tile(int op, int m, int n, int k, int num_cus, int* block_m, int* block_n) {
    if (!block_m || !block_n || num_cus <= 0) return 1;
    if (op == 0) {
        if (const int atoms = dense_skinny_atoms(m, n, k, num_cus)) { *block_m = 16 * atoms; *block_n = 16; }
        else pick(kDenseTiles, m, n, num_cus, block_m, block_n);
    }
    else if (op == 1) {
        if (const int atoms = skinny_atoms(m, n, num_cus)) { *block_m = 16 * atoms; *block_n = 16; }
        else pick(kFp8Tiles, m, n, num_cus, block_m, block_n);
    }
    else if (op == 2) pick_grouped(m, n, num_cus, 1, 128, k, block_m, block_n);
    else if (op == 3) { const yan::FloatTile t = yan::pick_float_tile(m, n, num_cus); *block_m = t.block_m; *block_n = t.block_n; }
    else if (op == 4) { const bool device = rows_on_device(m, n, num_cus, k); *block_m = device ? 256 : 0; *block_n = device ? 256 : 0; }
    else return 1;
    return 0;
}

int yan_gemm_select_split_k(int op, int m, int n, int k, int num_cus, int* block_m, int* block_n, int* split_k) {
    if (!block_m || !block_n || !split_k || num_cus <= 0 || (op != 0 && op != 1)) return 1;
    const bool split = op == 0 ? pick_dense_split_k(m, n, k, num_cus, block_m, block_n, split_k)
                               : pick_split_k(m, n, k, num_cus, block_m, block_n, split_k);
    if (!split) { *block_m = *block_n = 0; *split_k = 1; }
    return 0;
}

const char* yan_gemm_version(void) { return "yan-gemm gfx950 11 dense + 22 split-K dense + 2 weight-streaming dense + 7 fp32 + 10 fp8 tile variants + 15 split-K fp8 variants + 1 weight-streaming fp8 variant + 13 grouped fp8 variants + 4 quantiser kernels"; }

} // extern "C"
