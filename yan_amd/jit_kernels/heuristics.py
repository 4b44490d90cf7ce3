"""Macro-tile selection for a 256-CU part.

The reference leaves this open: its dense entry hard-codes one tile and an empty tuning space
(`yan/jit_kernels/cute_gemm.py:39-53`) and its FP8 template takes BLOCK_M / BLOCK_N as keys without saying who
picks them (`yan/jit_kernels/gemm.py:13-16`). Here a small cost model ranks the tiles the kernels support:
one workgroup per tile, one workgroup per CU at a time, so a launch costs
`ceil(tiles / num_cus)` rounds of one tile time, and a tile's time grows with its MFMA work but shrinks per
flop as the tile gets larger (fewer operand bytes fetched per flop).
"""
from typing import List, Optional, Tuple

from .utils import ceil_div

# (BLOCK_M, BLOCK_N): relative time per unit of tile area. Bigger tiles reuse operands better.
# Dense tiles: 256 rows x {256, 224, 192, 160} columns run the persistent 4-wave kernel with a ring of five LDS units (the
# 8-wave kernel on two stages for short or ragged K), the others the 4-wave kernel with a ring of stages. Costs of the 256-row
# tiles are measured: time per output of a problem that fills four whole rounds of 256 compute units with the tile
# (8192 x 32 BLOCK_N x 8192), relative to 256 x 256 (1.02-1.04, 1.035-1.06, 1.07-1.10 over three boxes). The ring tiles measure
# 1.30-1.32 (256 x 128, 128 x 256) and 1.49 (128 x 128) there, but no problem of four rounds ever takes them: where they
# compete, in launches of one or two rounds, a tile pays its first loads and its epilogue in full, and 1.40 / 1.42 is what
# makes the table's pick the fastest tile or within 1.2 % of it on all 67 shapes swept with every tile forced in turn (with
# 1.30, 128 x 256 took eight one-round shapes from 256 x 160, which is 4 to 17 % faster there).
# 128 x 192 and 64 x 192 (ring kernel, wave slabs 96 columns wide) are for problems that leave most compute units idle with
# 256-wide tiles and need two rounds with 128-wide ones (2048 x 2112 x 7168: 144 tiles of 128 x 256 run 85 us, 176 of 128 x 192 68 us).
_DENSE_TILES = {(256, 256): 1.00, (256, 224): 1.03, (256, 192): 1.05, (256, 160): 1.085, (256, 128): 1.42, (128, 256): 1.40,
                (128, 192): 1.43, (128, 128): 1.51, (64, 192): 1.96, (64, 128): 2.0, (64, 64): 2.78}
# FP8 tiles: measured over 74 shapes (m = 17 ... 8192, n = 2048 ... 32768, k = 512 ... 16384) with every tile forced in turn;
# with these costs the model's pick is within 1 % of the fastest tile on all of them. 256 x 192 and 256 x 160 are there for
# problems whose 256 x 256 tiles leave a round of compute units partly empty (4096 x 5120 x 5120: 320 tiles, against 512
# tiles of 256 x 160 = two full rounds, 13 % faster); 256 x 224 and 64 x 160 are supported by the kernel and never the
# cheapest (a round of 64 x 160 tiles takes longer than a round of 128 x 128 tiles, which run eight waves).
_FP8_TILES = {(256, 256): 1.00, (256, 192): 1.12, (256, 160): 1.28, (256, 128): 1.34, (128, 256): 1.34, (128, 128): 1.5,
              (64, 128): 2.3, (64, 64): 3.55, (64, 32): 4.8, (32, 32): 7.0}


def rank_tiles(m: int, n: int, num_cus: int, table, groups: int = 1) -> List[Tuple[float, Tuple[int, int]]]:
    ranked = []
    for (bm, bn), per_area in table.items():
        tiles = ceil_div(m, bm) * ceil_div(n, bn) * groups
        rounds = ceil_div(tiles, num_cus)
        ranked.append((rounds * bm * bn * per_area, (bm, bn)))
    return sorted(ranked)


def tuning_enabled() -> bool:
    """Empirical tile selection on the first call per shape (`YAN_TUNE_TILES=1`): the entry points hand the cost model's
    three best tiles to the tuner as its `space` and the fastest on the device wins, as the reference's tuner does with
    its candidate list (`yan/jit_kernels/cute_gemm.py:42-53`, `tuner.py:42-69`). Off by default: the first call of a
    shape then costs up to three compilations and sixty timed launches."""
    import os
    return os.getenv('YAN_TUNE_TILES', '0') not in ('', '0')


def get_dense_tile_space(m: int, n: int, k: int, num_cus: int, count: int = 3) -> List[Tuple[int, int]]:
    return [tile for _, tile in rank_tiles(m, n, num_cus, _DENSE_TILES)[:count]]


def get_fp8_tile_space(m: int, n: int, k: int, num_cus: int, count: int = 3) -> List[Tuple[int, int]]:
    return [tile for _, tile in rank_tiles(m, n, num_cus, _FP8_TILES)[:count]]


def get_best_dense_config(m: int, n: int, k: int, num_cus: int) -> Tuple[int, int]:
    return rank_tiles(m, n, num_cus, _DENSE_TILES)[0][1]


def get_best_fp8_config(m: int, n: int, k: int, num_cus: int) -> Tuple[int, int]:
    return rank_tiles(m, n, num_cus, _FP8_TILES)[0][1]


def get_dense_num_stages(block_m: int, block_n: int) -> int:
    """LDS stages of the dense kernel for a tile: 2 names the persistent kernels of the tiles with 256 rows and more than 128
    columns (8 waves on two stages, or 4 waves on a ring of five operand units for 256 x 256: the launcher chooses), else as
    many as the 160 KB LDS holds, at most 8 (`DenseTileConfig::MAX_STAGES` in bf16_gemm.hpp): 3 for 128 x 256, ... 8 for 64 x 64."""
    if block_m == 256 and block_n > 128:
        return 2            # the persistent kernels, whatever the width
    return min(8, 160 * 1024 // ((block_m + block_n) * 128))


def get_fp8_num_stages(block_m: int, block_n: int) -> int:
    """LDS stages of the tiled FP8 kernel for a tile: a ring as deep as the 160 KB LDS allows, at most 8, or 12 for the
    tiles of 32 weight rows that run the decode shapes (`Fp8TileConfig::MAX_RING_STAGES` in fp8_gemm.hpp): 2 for
    256 x 256, 3 for 256 x 128 and 128 x 256, 8 for 64 x 64, 12 for 64 x 32 and 32 x 32. Tiles below 256 x 256 are what the cost model picks when a problem is short on work per CU, i.e. bound by
    operand streaming, and there one k-tile of prefetch does not cover the memory latency."""
    waves = 4               # get_num_waves in mfma_utils.hpp
    if block_m * block_n >= 256 * 128 or (block_m * block_n >= 64 * 64 and block_m % 64 == 0 and block_n % 64 == 0):
        waves = 8
    capable = block_m % 32 == 0 and (block_m // 8) % waves == 0 and block_n % 16 == 0
    if not capable:
        return 2
    rows = ceil_div(block_m, 8 * waves) * 8 * waves + ceil_div(block_n, 8 * waves) * 8 * waves      # whole copy passes
    stage_bytes = rows * 128 + ceil_div(block_m * 4, 1024) * 1024
    return max(2, min(12 if block_n <= 32 else 8, 160 * 1024 // stage_bytes))


def get_best_grouped_fp8_config(m: int, n: int, k: int, num_cus: int, groups: int = 1, m_alignment: int = 0,
                                groups_in_m: int = 1) -> Tuple[int, int]:
    """Tile of a grouped FP8 GEMM, among the tiles 64, 128 or 256 columns wide. Contiguous layout: `m` is the total row count, `m_alignment` the padding of every
    group and `groups_in_m` the number of groups sharing the rows: a tile of up to `m_alignment` rows must divide it;
    the 256-row tile, which handles a group boundary in its middle with a second pass over K, is offered when groups
    average at least 1024 rows. Masked layout: `m` is the expected row count of one group and `groups` multiplies
    the tile count."""
    def allowed(bm):
        if m_alignment == 0 or m_alignment % bm == 0:
            return True
        return bm == 2 * m_alignment and m >= 1024 * groups_in_m
    table = {t: c for t, c in _FP8_TILES.items() if t[1] in (64, 128, 256) and allowed(t[0])}
    return rank_tiles(max(m, 1), n, num_cus, table, groups)[0][1]


def get_contiguous_rows_on_device(m: int, n: int, k: int, num_cus: int, groups_in_m: int) -> bool:
    """Whether a contiguous grouped GEMM runs the kernel that decides on the device what its 256-row tiles do about group
    boundaries (`fp8_gemm_contiguous_rows_kernel`): groups of 256 to 2047 rows on average for which the cost table, with
    256-row tiles allowed, takes 256 x 256 tiles. Which tile rows hold two groups stands in `m_indices`: with none (every
    boundary on a multiple of 256 rows) 256-row tiles are 13-17 % faster than 128 x 256 ones (16 groups of 512 rows x 4096 x
    7168: 225 against 264 us), with a few the kernel runs those rows as 128-row tiles at the end of the launch (8 groups
    of 896 and 1152 rows: 230 against 250 us with two-pass tiles), with many it runs 128-row tiles throughout. Longer groups keep
    the fixed 256-row tiles (within 2 % either way, and the fixed kernel is the faster when no row holds two groups). Same
    rule as `rows_on_device` in yan_amd/csrc/yan_gemm_capi.hip."""
    if groups_in_m <= 0 or not 256 * groups_in_m <= m < 2048 * groups_in_m:
        return False
    table = {t: c for t, c in _FP8_TILES.items() if t[1] in (64, 128, 256) and t[0] in (64, 128, 256)}
    return rank_tiles(m, n, num_cus, table)[0][1] == (256, 256)


def get_skinny_fp8_config(m: int, n: int, k: int, num_cus: int) -> int:
    """Number of 16-row activation atoms (1) when the weight-streaming kernel should run instead of the tiled one, else 0:
    up to 16 activation rows, and few enough weight rows that its n/16 workgroups fit the chip in one round. Measured
    on 256 CUs (kernel time warm / after a cache flush, weight-streaming vs tiled with its ring of LDS stages):
    m = 1..16, n = 4096, k = 7168: 7.4-9.3 / 13.4 us vs 13.7-14.0 / 15.3 us; n = 2048: 6.9-9.1 / 9.4-10.4 vs 13.6 / 14.4;
    n = 7168: 12.9-15.5 / 22 vs 15.5 / 21 (a tie, and two rounds of workgroups). From 17 rows up the tiled kernel wins or
    ties everywhere (m = 64, n = 4096, k = 7168: 14.5 / 17.2 us)."""
    if 0 < m <= 16 and 16 <= n <= 16 * num_cus:
        return 1
    return 0


def get_skinny_dense_config(m: int, n: int, k: int, num_cus: int) -> int:
    """Number of 16-row activation atoms (1 or 2) when the weight-streaming dense kernel should run instead of the tiled
    one, else 0: up to 32 activation rows, few enough weight rows that its n/16 workgroups fit the chip in one round, and
    whole 128-byte K blocks. The smallest dense tile gives a workgroup 64 weight rows: n = 4096 puts 64 of 256 compute
    units to work. Measured call to call with the weights cycling through more matrices than the caches hold (bf16,
    n = 4096, k = 7168; weight-streaming vs 64 x 64 tiles): m = 1: 14.5 vs 25.9 us, m = 16: 18.3 vs 27.0, m = 17: 21.3 vs
    27.1, m = 32: 25.4 vs 30.1, m = 48: 30.7 vs 33.3 (three atoms: not offered), m = 64: a tie; n = 2112 alike. Beyond one
    round of workgroups the tiles win (n = 7168, k = 2048: 11.7 vs 10.2 us at m = 1; n = 16384, k = 4096: 34.0 vs 30.7),
    and two atoms lose on short K (k = 1024: 7.2 vs 6.0 us)."""
    if n < 16 or n > 16 * num_cus or n % 4 or k <= 0 or k % 64:
        return 0
    if 0 < m <= 16:
        return 1
    if 16 < m <= 32 and k >= 2048:
        return 2
    return 0


def get_dense_tile(m: int, n: int, k: int, num_cus: int) -> Tuple[int, int]:
    """(BLOCK_M, BLOCK_N) of the dense kernel that runs: (16 * atoms, 16) for the weight-streaming kernel."""
    atoms = get_skinny_dense_config(m, n, k, num_cus)
    return (16 * atoms, 16) if atoms else get_best_dense_config(m, n, k, num_cus)


def get_fp8_tile(m: int, n: int, k: int, num_cus: int) -> Tuple[int, int]:
    """(BLOCK_M, BLOCK_N) of the FP8 kernel that runs: (16 * atoms, 16) for the weight-streaming kernel."""
    atoms = get_skinny_fp8_config(m, n, k, num_cus)
    return (16 * atoms, 16) if atoms else get_best_fp8_config(m, n, k, num_cus)


# Split-K of the FP8 GEMM: microseconds a workgroup spends per k-tile on a ring tile when every compute unit runs one
# (measured: m x 4096 x 7168, sizes at run time, 56 k-tiles, one round of workgroups). Only used to weigh split-K plans
# against the unsplit pick of the cost table above.
_FP8_SPLIT_K_TILE_US = {(32, 32): 0.133, (64, 32): 0.192, (64, 64): 0.296, (64, 128): 0.395, (128, 128): 0.51}
# The same for the unsplit kernel, which pulls its weights with fewer workgroups at a time and, a workgroup per tile, runs
# without a loop around the tile: 0.88 to 0.975 of the figures above.
_FP8_UNSPLIT_TILE_US = {(32, 32): 0.117, (64, 32): 0.169, (64, 64): 0.275, (64, 128): 0.375, (128, 128): 0.497}
FP8_SPLIT_K_FACTORS = (2, 3, 4)


def get_split_k_fp8_config(m: int, n: int, k: int, num_cus: int) -> Optional[Tuple[int, int, int]]:
    """(BLOCK_M, BLOCK_N, SPLIT_K) when the plain FP8 GEMM should split K over SPLIT_K workgroups per tile, else None.

    A problem whose unsplit tiles fit the chip in one round is bound by what one compute unit can pull per k-tile
    (60-65 GB/s whatever the tile), and every workgroup pulls the activation rows of its tile over all of K. With K split,
    a larger tile on as many workgroups pulls fewer bytes per output; the price is a round trip of the partial sums
    through memory, paid by the part that arrives last. Modelled time of a plan: k-tiles per part x the tile's time per
    k-tile + 0.5 us + 12.5 ns per KB of partial sums the last part reads, never less than streaming the weights at 6 TB/s.
    A plan is taken when it fits one round (tile slots x SPLIT_K <= num_cus), leaves every part at least 14 k-tiles (24 when there are only two parts) and beats
    the unsplit pick (its own, slightly lower time per k-tile) by a tenth of its modelled time plus 3.5 us of launch. On 36 shapes (m = 32..256, n = 1536..24576,
    k = 1536..16384) swept with every tile and factor, weights cycling through more matrices than the caches hold, the
    plan taken is the fastest measured or within 1 % of it wherever one is taken (64 x 4096 x 7168: 64 x 64 tiles in four
    parts; 32 x 2112 x 7168: 32 x 32 in three); over 80 shapes with a plan (m = 17..1024, 13 (n, k)) it takes 0.47 to 1.04 of the
    unsplit time, median 0.83; k up to about 5000 in two parts, k = 2048 and n = 16384 or more stay unsplit. A plan also goes before the weight-streaming kernel of up to 16 rows (32 x 32 tiles in two to four parts
    against that kernel, m = 1..16: n = 4096, k = 7168: 9.7 - 9.8 against 10.7 - 12.2 us; n = 2048: 8.4 against 10.1 - 11.8; level
    at k = 4096 and at k = 16384 below 8 rows), which runs where no plan exists or no workspace is at hand. Same rule as
    `pick_split_k` in yan_amd/csrc/yan_gemm_capi.hip (a CPU test keeps the two in step)."""
    if m <= 0 or n <= 0:
        return None
    k_tiles = k // 128
    unsplit = get_best_fp8_config(m, n, k, num_cus)
    if unsplit not in _FP8_SPLIT_K_TILE_US or ceil_div(m, unsplit[0]) * ceil_div(n, unsplit[1]) > num_cus:
        return None
    floor = n * k / 6.0e6
    base = max(k_tiles * _FP8_UNSPLIT_TILE_US[unsplit], floor)
    best, best_plan = None, None
    for (bm, bn), per_k_tile in _FP8_SPLIT_K_TILE_US.items():
        if bm > 32 and bm >= 2 * m:
            continue                # a tile more than twice as tall as the problem
        tiles = ceil_div(m, bm) * ceil_div(n, bn)
        for split in FP8_SPLIT_K_FACTORS:
            # a workgroup per part of every tile slot (tiles rounded up to the 8 XCDs); 256 also bounds the workspace
            # two parts save half the k-tiles at most: they pay from 24 k-tiles per part on, three and four from 14
            if ceil_div(tiles, 8) * 8 * split > min(num_cus, 256) or ceil_div(k_tiles, split) < (24 if split == 2 else 14):
                continue
            t = max(ceil_div(k_tiles, split) * per_k_tile + 0.5 + (split * bm * bn * 4) / 1024 * 0.0125, floor)
            if best is None or t < best:
                best, best_plan = t, (bm, bn, split)
    if best is not None and base - best >= 0.10 * (base + 3.5):
        return best_plan
    return None


# Split-K of the dense GEMM: microseconds per k-tile (64 deep) of a workgroup on a ring tile with the chip full (measured with
# weights cycling through more matrices than the caches hold), for every tile the unsplit pick can be; the first three are
# the tiles split-K plans use, with what their longer ring fill and larger partial sums add per launch.
_DENSE_SPLIT_K_TILE_US = {(64, 64): 0.248, (64, 128): 0.378, (128, 128): 0.51, (64, 192): 0.60, (128, 192): 0.80, (128, 256): 0.94,
                          (256, 128): 0.94}
_DENSE_SPLIT_K_EXTRA_US = {(64, 64): 0.0, (64, 128): 1.0, (128, 128): 2.5}
DENSE_SPLIT_K_FACTORS = (2, 3, 4, 6, 8)         # six and eight parts on 64 x 64 tiles only (few weight rows, long K)


def get_split_k_dense_config(m: int, n: int, k: int, num_cus: int) -> Optional[Tuple[int, int, int]]:
    """(BLOCK_M, BLOCK_N, SPLIT_K) when the dense 16-bit GEMM should split K over SPLIT_K workgroups per tile, else None.
    The rule of `get_split_k_fp8_config` with the dense tiles' numbers: the smallest dense tile holds 64 weight rows, so
    m = 64, n = 4096 puts 64 of 256 compute units to work and K = 7168 keeps each for 112 k-tiles; in four parts the same
    tiles fill the chip. A plan fits one round (tile slots x SPLIT_K <= num_cus), leaves every part at least 16 k-tiles and
    must beat the unsplit pick by 11 % of its modelled time plus 3.5 us. Measured (bf16, weights cycling, unsplit ->
    plan): 64 x 4096 x 7168 37.1 -> 16.2 us, 256 x 2048 x 7168 34.2 -> 20.3, 256 x 5120 x 5120 44.7 -> 33.9,
    64 x 2048 x 7168 36.1 -> 12.8 (six parts; four: 14.5), 64 x 1024 x 16384 69.3 -> 16.5 (eight parts; four: 24.1),
    256 x 7168 x 16384 113.4 -> 90.9, 512 x 4096 x 7168 53.4 -> 43.9 (hipBLASLt on the first five and the 256-row shapes: 22.7, 24.7, 49.6, 140.4);
    over 54 shapes swept with every tile and factor the plan is the fastest measured or within 6 % of it (11 % in one case),
    and over 118 shapes with a plan (m = 33..1024, 14 (n, k)) it takes 0.35 to 0.92 of the unsplit time, median 0.65. Same rule as
    `pick_dense_split_k` in yan_amd/csrc/yan_gemm_capi.hip (a CPU test keeps the two in step). A plan goes before the
    two-atom weight-streaming kernel (17 to 32 rows; n = 4096, k = 7168: 21.1 - 25.2 us against 14.8 - 14.9 for 64 x 64 tiles
    in four parts), which therefore runs only where no plan exists or no workspace is at hand (the C library's plain entry
    points), and before the one-atom kernel from 8 rows on K up to 8192 (m = 8: 15.8 against 14.7 us, m = 16: 18.2 against 14.8;
    n = 2048: 15.0 / 17.5 against 12.3 / 12.4); below 8 rows and on longer K that kernel stays (m = 1: 14.5 against 14.7;
    k = 16384, m = 8: 28.9 against 31.0)."""
    if m <= 0 or n <= 0 or k <= 0 or ((m < 8 or (m <= 16 and k > 8192)) and get_skinny_dense_config(m, n, k, num_cus)):
        return None         # a handful of rows, or up to 16 on a long K: the one-atom weight-streaming kernel is as fast or faster
    k_tiles = ceil_div(k, 64)
    unsplit = get_best_dense_config(m, n, k, num_cus)
    if unsplit not in _DENSE_SPLIT_K_TILE_US or ceil_div(m, unsplit[0]) * ceil_div(n, unsplit[1]) > num_cus:
        return None
    floor = n * k * 2 / 6.0e6
    base = max(k_tiles * _DENSE_SPLIT_K_TILE_US[unsplit], floor)
    best, best_plan = None, None
    for (bm, bn), extra in _DENSE_SPLIT_K_EXTRA_US.items():
        if bm > 64 and bm >= 2 * m:
            continue                # a tile more than twice as tall as the problem
        tiles = ceil_div(m, bm) * ceil_div(n, bn)
        for split in DENSE_SPLIT_K_FACTORS:
            if split > 4 and (bm, bn) != (64, 64):
                continue            # the last part of a larger tile would hold more partial sums than it has registers for
            if ceil_div(tiles, 8) * 8 * split > min(num_cus, 256) or ceil_div(k_tiles, split) < 16:
                continue
            t = max(ceil_div(k_tiles, split) * _DENSE_SPLIT_K_TILE_US[(bm, bn)] + 0.5 + (split * bm * bn * 4) / 1024 * 0.0125 + extra, floor)
            if best is None or t < best:
                best, best_plan = t, (bm, bn, split)
    if best is not None and base - best >= 0.11 * (base + 3.5):
        return best_plan
    return None


# (BLOCK_M, BLOCK_N) -> cost per unit of tile area; tiles below 128 rows split K over their four waves.
_FLOAT_TILES = {(256, 256): 1.00, (128, 256): 1.015, (128, 128): 1.03, (128, 64): 1.04, (64, 64): 1.13, (32, 64): 1.13, (32, 32): 1.25}


def get_best_float_config(m: int, n: int, num_cus: int) -> Tuple[int, int]:
    """(BLOCK_M, BLOCK_N) of the fp32 GEMM: rounds of workgroups over the CUs times the tile's area times its cost
    per area; ties go to the earlier, larger tile. Same table and rule as `yan::pick_float_tile` in
    gemm/simple_gemm.hpp (a CPU test keeps the two in step)."""
    best, best_cost = None, None
    for (bm, bn), per_area in _FLOAT_TILES.items():
        tiles = ceil_div(m, bm) * ceil_div(n, bn)
        cost = ceil_div(tiles, num_cus) * bm * bn * per_area
        if best_cost is None or cost < best_cost:
            best, best_cost = (bm, bn), cost
    return best
