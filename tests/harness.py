"""Harness-side helpers shared by the tests, the smoke entry and the benchmark (not part of the operator package): FP8 quantisers in the DeepGEMM
convention and seeded constructors for the benchmark configurations. The reference defines neither (its FP8 path
has no Python entry or test); the recipes are the ones the benchmark configurations name:
per-token 1x128 / per-block 128x128 amax, clamp 1e-4, x * (448 / amax) -> e4m3fn, scale = amax / 448.
Both quotients are tensor / tensor divisions on purpose: torch turns `448.0 / amax` into reciprocal(amax) * 448 and,
on the GPU, `amax / 448.0` into amax * (1 / 448), each an ulp away from the correctly rounded quotient for some inputs.
"""
from typing import Tuple

import torch

FP8_MAX = 448.0


def per_token_cast_to_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """x [m, k] (k % 128 == 0) -> (e4m3fn [m, k], fp32 scales [m, k/128])."""
    assert x.dim() == 2 and x.size(1) % 128 == 0
    m, k = x.shape
    xv = x.float().view(m, k // 128, 128)
    amax = xv.abs().amax(dim=2).clamp(1e-4)
    top = torch.full_like(amax, FP8_MAX)
    q = (xv * (top / amax).unsqueeze(2)).to(torch.float8_e4m3fn)
    return q.view(m, k), amax / top


def per_block_cast_to_fp8(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """w [n, k] (k % 128 == 0) -> (e4m3fn [n, k], fp32 scales [ceil(n/128), k/128])."""
    assert w.dim() == 2 and w.size(1) % 128 == 0
    n, k = w.shape
    n_pad = (n + 127) // 128 * 128
    wp = torch.zeros((n_pad, k), dtype=torch.float32, device=w.device)
    wp[:n] = w
    wv = wp.view(n_pad // 128, 128, k // 128, 128)
    amax = wv.abs().amax(dim=(1, 3)).clamp(1e-4)
    top = torch.full_like(amax, FP8_MAX)
    q = (wv * (top / amax)[:, None, :, None]).to(torch.float8_e4m3fn)
    return q.view(n_pad, k)[:n].contiguous(), amax / top


def dequant_lhs(q: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    return q.float() * scales.repeat_interleave(128, dim=1)


def dequant_rhs(q: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    n = q.size(0)
    return q.float() * scales.repeat_interleave(128, dim=0)[:n].repeat_interleave(128, dim=1)


def _source(rows: int, cols: int, dist: str, gen: torch.Generator, device) -> torch.Tensor:
    if dist == 'normal':
        return torch.randn(rows, cols, generator=gen, device=device)
    if dist == 'outlier':     # uniform[-4, 4] with 1% of the entries multiplied by 50
        x = torch.rand(rows, cols, generator=gen, device=device) * 8 - 4
        hot = torch.rand(rows, cols, generator=gen, device=device) < 0.01
        return torch.where(hot, x * 50, x)
    raise ValueError(dist)


def make_bf16_case(m: int, n: int, k: int, seed: int = 42, scale: float = 1.0, dtype=torch.bfloat16,
                   device='cpu', gen_device='cpu'):
    """A [m,k], B [n,k] ~ N(0,1)*scale in `dtype`, plus a zeroed C [m,n]. Values are drawn on `gen_device`
    (CPU by default so that host and GPU paths see the same bits) and moved to `device`."""
    gen = torch.Generator(device=gen_device).manual_seed(seed)
    a = (torch.randn(m, k, generator=gen, device=gen_device) * scale).to(dtype).to(device)
    b = (torch.randn(n, k, generator=gen, device=gen_device) * scale).to(dtype).to(device)
    return a, b, torch.zeros(m, n, dtype=dtype, device=device)


def make_float_case(m: int, n: int, k: int, seed: int = 42, device='cpu', gen_device='cpu'):
    """A [m,k] and B [n,k] ~ N(0,1) in fp32, stored with their first dimension contiguous (what `gemm_float_nt`
    takes), plus a zeroed row-major C [m,n]."""
    gen = torch.Generator(device=gen_device).manual_seed(seed)
    a = torch.randn(k, m, generator=gen, device=gen_device).to(device).t()
    b = torch.randn(k, n, generator=gen, device=gen_device).to(device).t()
    return a, b, torch.zeros(m, n, dtype=torch.float32, device=device)


def make_fp8_case(m: int, n: int, k: int, seed: int = 42, dist: str = 'normal', device='cpu', gen_device='cpu',
                  col_major_scales: bool = False):
    """((A8, sA), (B8, sB), out) for the block-scaled GEMM, quantised from seeded fp32 sources.
    Sources are drawn and quantised in row slabs so that the 16384^3 case never holds two fp32 matrices."""
    gen = torch.Generator(device=gen_device).manual_seed(seed)

    def build(rows, quantise, align):
        qs, ss = [], []
        step = max(align, (1 << 26) // k // align * align)
        for r0 in range(0, rows, step):
            r = min(step, rows - r0)
            q, s = quantise(_source(r, k, dist, gen, gen_device).to(device))
            qs.append(q), ss.append(s)
        return torch.cat(qs), torch.cat(ss)

    a8, sa = build(m, per_token_cast_to_fp8, 1)
    b8, sb = build(n, per_block_cast_to_fp8, 128)
    if col_major_scales:
        from yan_amd.jit_kernels.utils import get_col_major_tensor
        sa = get_col_major_tensor(sa)
    return (a8, sa), (b8, sb), torch.zeros(m, n, dtype=torch.bfloat16, device=device)


def make_grouped_contiguous_case(group_rows, n: int, k: int, seed: int = 42, device='cpu', gen_device='cpu',
                                 padding_blocks: int = 0, alignment: int = 128):
    """((A8, sA), (B8 [G,n,k], sB [G,ceil(n/128),k/128]), out, m_indices) for the contiguous grouped layout:
    the g-th positive entry of `group_rows` is group g and contributes that many real rows, padded with zero rows up to
    the alignment (padding rows carry the group's index, as a caller that pads with zeros would do); a negative entry
    is a block of that many padding rows (index -1, a multiple of the alignment) at that position; `padding_blocks`
    whole blocks with index -1 follow at the end. Padding blocks hold random values, which the kernel must not touch.
    `out` is pre-filled with a sentinel so that rows the kernel must not write can be checked."""
    groups = sum(1 for r in group_rows if r > 0)
    gen = torch.Generator(device=gen_device).manual_seed(seed)
    qs, ss, idx = [], [], []
    g = 0
    for rows in tuple(group_rows) + ((-padding_blocks * alignment,) if padding_blocks else ()):
        if rows > 0:
            padded = (rows + alignment - 1) // alignment * alignment
            x = torch.zeros(padded, k, device=gen_device)
            x[:rows] = torch.randn(rows, k, generator=gen, device=gen_device)
            label, g = g, g + 1
        else:
            padded = -rows
            assert padded % alignment == 0
            x = torch.randn(padded, k, generator=gen, device=gen_device)
            label = -1
        q, sc = per_token_cast_to_fp8(x.to(device))
        qs.append(q), ss.append(sc), idx.append(torch.full((padded,), label, dtype=torch.int32))
    a8, sa = torch.cat(qs), torch.cat(ss)
    ws = [per_block_cast_to_fp8(torch.randn(n, k, generator=gen, device=gen_device).to(device)) for _ in range(groups)]
    b8, sb = torch.stack([w[0] for w in ws]), torch.stack([w[1] for w in ws])
    out = torch.full((a8.size(0), n), -7.0, dtype=torch.bfloat16, device=device)
    return (a8, sa), (b8, sb), out, torch.cat(idx).to(device)


def make_grouped_masked_case(groups: int, m_max: int, n: int, k: int, masked, seed: int = 42, device='cpu', gen_device='cpu'):
    """((A8 [G,m_max,k], sA [G,m_max,k/128]), (B8 [G,n,k], sB), out [G,m_max,n], masked_m) for the masked layout;
    `out` is pre-filled with a sentinel."""
    gen = torch.Generator(device=gen_device).manual_seed(seed)
    xs = [per_token_cast_to_fp8(torch.randn(m_max, k, generator=gen, device=gen_device).to(device)) for _ in range(groups)]
    ws = [per_block_cast_to_fp8(torch.randn(n, k, generator=gen, device=gen_device).to(device)) for _ in range(groups)]
    a8, sa = torch.stack([x[0] for x in xs]), torch.stack([x[1] for x in xs])
    b8, sb = torch.stack([w[0] for w in ws]), torch.stack([w[1] for w in ws])
    out = torch.full((groups, m_max, n), -7.0, dtype=torch.bfloat16, device=device)
    return (a8, sa), (b8, sb), out, torch.tensor(list(masked), dtype=torch.int32, device=device)


# ----------------------------------------------------------------------------- shapes exercised on the GPU
# (m, n, k). Listed here so that every JIT kernel they need can be compiled ahead of time, without a GPU.
BASELINE_BF16 = {'cfg1': (1024, 1024, 1024), 'cfg2': (8192, 8192, 8192)}
BASELINE_FP8 = {'cfg3': (4096, 7168, 7168), 'cfg4': (64, 4096, 7168), 'cfg5': (16384, 16384, 16384)}

DENSE_TEST_SHAPES = [
    (1024, 1024, 1024), (8192, 8192, 8192),
    (128, 256, 256), (64, 64, 64), (1, 64, 64), (255, 132, 72), (300, 520, 8), (33, 4, 200), (257, 1028, 1096),
    (300, 256, 256), (33, 132, 72), (96, 80, 136),
    (256, 5120, 5120), (4096, 2048, 7168), (4096, 7168, 2048), (256, 24576, 1536),
    (128, 4096, 7168), (512, 4096, 2048), (1024, 7168, 1024),
    (3000, 5000, 1000),          # the 256 x 256 tile (8-wave kernel: K is not whole k-tiles) with ragged m, n and a k tail
    (2900, 5004, 520),           # same with n % 8 == 4 (narrow stores) and an odd number of k-tiles
    (2900, 5000, 64),            # same with a single k-tile
    (3000, 5000, 960),           # the 256 x 256 tile on the 4-wave kernel (whole k-tiles, an odd number of them), ragged m and n
    (2900, 5000, 256),           # same with four k-tiles, the fewest it takes
    # the narrower tiles of 256 rows: 256 x 160, 256 x 224, 256 x 192, each once whole (4-wave kernel) and once ragged in m, n
    # and k (8-wave kernel)
    (4096, 5120, 512), (4000, 5000, 520), (2048, 7168, 256), (2047, 7100, 264), (4096, 6144, 256), (4090, 6100, 72),
    # and ragged in m and n on the 4-wave kernel (whole k-tiles, n a multiple of 8)
    (4000, 5000, 576), (2047, 7096, 832), (4090, 6104, 320),
    # the 192-wide tiles of the ring kernel (wave slabs of 96 columns), whole and ragged
    (2048, 2112, 264), (2000, 2100, 136), (1024, 2112, 264), (1000, 2100, 72),
    # a handful of rows over up to 4096 weight rows: the weight-streaming kernel with one and two activation atoms, the
    # last workgroup partly past n, fewer K blocks than waves ((1, 64, 64) above), more than one pass over the waves
    (1, 4096, 7168), (16, 2112, 1024), (7, 1156, 512), (17, 4096, 2048), (32, 272, 4096), (20, 100, 2112),
]
# Shapes for every 256-row tile width in turn, with the tile given (whatever the cost model would pick): the edges of what the
# 4-wave kernel takes (four k-tiles, eight columns, one row) and seeded random ones; n a multiple of 8 and K whole k-tiles.
def _seeded_dense_shapes(count, seed=7):
    import random
    rng = random.Random(seed)
    return [(rng.randint(1, 6000), 8 * rng.randint(1, 800), 64 * rng.randint(4, 40)) for _ in range(count)]


DENSE_SEEDED_BOTH_KERNELS_SHAPES = [(1, 8, 256), (255, 160, 256), (257, 168, 320), (5000, 8, 2560), (1, 6000, 1024), (4097, 4104, 256)] + _seeded_dense_shapes(8)
# (shape, tile the cost model must pick): the shapes above exist for these tiles
DENSE_TILE_OF_SHAPE = {(4096, 5120, 512): (256, 160), (4000, 5000, 520): (256, 160), (2048, 7168, 256): (256, 224),
                       (2047, 7100, 264): (256, 224), (4096, 6144, 256): (256, 192), (4090, 6100, 72): (256, 192),
                       (4000, 5000, 576): (256, 160), (2047, 7096, 832): (256, 224), (4090, 6104, 320): (256, 192),
                       (3000, 5000, 1000): (256, 256), (8192, 8192, 8192): (256, 256), (3000, 5000, 960): (256, 256), (2900, 5000, 256): (256, 256),
                       (2048, 2112, 264): (128, 192), (2000, 2100, 136): (128, 192), (1024, 2112, 264): (64, 192), (1000, 2100, 72): (64, 192),
                       (1, 4096, 7168): (16, 16), (7, 1156, 512): (16, 16), (17, 4096, 2048): (32, 16), (20, 100, 2112): (32, 16)}
# Shapes on which the launcher of the 256-row tiles takes the 4-wave kernel (whole k-tiles, at least four of them, n a multiple
# of 8), one or two per tile width; the 8-wave kernel of the same tile is built with explicit keys to compare bits.
DENSE_BOTH_KERNELS_SHAPES = [(3000, 5000, 960), (2900, 5000, 256), (3840, 4096, 576), (4096, 4096, 2048),
                             (4096, 5120, 512), (4000, 5000, 576), (2047, 7096, 832), (4090, 6104, 320)]


def dense_explicit_plan(tile, dtype=torch.bfloat16, eight_waves: bool = False):
    """(name, keys, arg_defs, template) of a dense kernel with the tile given; `eight_waves` names the 8-wave kernel of a
    256-row tile whatever the shape."""
    from yan_amd.jit_kernels import bf16_gemm
    from yan_amd.jit_kernels.heuristics import get_dense_num_stages
    keys = {'BLOCK_M': tile[0], 'BLOCK_N': tile[1], 'NUM_STAGES': get_dense_num_stages(*tile), 'NUM_SMS': 0}
    template = bf16_gemm.template
    if eight_waves:
        assert tile[0] == 256 and tile[1] >= 160 and 'gemm_tn<BLOCK_M, BLOCK_N, kNumStages>' in template
        template = template.replace('gemm_tn<BLOCK_M, BLOCK_N, kNumStages>', 'gemm_tn<BLOCK_M, BLOCK_N, kNumStages, 8>')
    name = ('gemm_bf16_tn' if dtype == torch.bfloat16 else 'gemm_fp16_tn') + ('_eight_waves' if eight_waves else '')
    return name, keys, bf16_gemm._arg_defs(dtype), template


# (m, n, k) of the reference's own dense test (tests/test_cute.py:21-22: m in (256, 4096) x six (k, n) pairs)
REFERENCE_DENSE_TEST_SHAPES = [(m, n, k) for m in (256, 4096)
                               for k, n in ((5120, 5120), (1536, 24576), (512, 32768), (16384, 7168), (7168, 2048), (2048, 7168))]
# (m, n, k) of the reference's fp32 test (tests/test_simple.py:22-23: m in (128, 4096) x six (k, n) pairs)
REFERENCE_FLOAT_TEST_SHAPES = [(m, n, k) for m in (128, 4096)
                               for k, n in ((7168, 2112), (1536, 24576), (512, 32768), (16384, 7168), (7168, 4096), (2048, 7168))]
# small fp32 cases compared in full: k tails, and with the reference's shapes every tile variant (32x32, 32x64 and
# 64x64 with K split over the waves; 128x64, 128x128, 128x256, 256x256)
FLOAT_TEST_SHAPES = [(128, 64, 16), (128, 64, 1), (128, 192, 17), (256, 320, 100), (384, 1024, 260), (128, 24576, 40),
                     (512, 4096, 40), (256, 32768, 24), (4096, 32768, 8)]
FP8_TEST_SHAPES = [
    (4096, 7168, 7168), (64, 4096, 7168), (16384, 16384, 16384),
    (64, 256, 384), (512, 1024, 1024), (1, 128, 128), (63, 192, 256), (129, 320, 128), (300, 96, 640),
    (40, 192, 256), (130, 448, 640),
    (257, 2112, 1024), (128, 7168, 2048), (4096, 2048, 7168),
    (1, 4096, 7168), (17, 4096, 1024), (33, 2112, 640), (64, 7168, 2048), (48, 4100, 384), (40, 2112, 640),
    (128, 4096, 7168), (512, 4096, 2048), (1024, 7168, 1024),
    # the 256-row tiles narrower than 256 columns, whole and ragged (FP8_TILE_OF_SHAPE below)
    (4096, 5120, 256), (4000, 5100, 384), (512, 24576, 256), (500, 24500, 384), (768, 10880, 256),
    (1024, 2112, 256), (1000, 2100, 384),
]
# Which tile the cost model picks for some of the shapes above on 256 compute units: a CPU test keeps this true, so that a
# change of the cost table cannot silently take a tile out of the parity tests.
FP8_TILE_OF_SHAPE = {(1024, 2112, 256): (128, 128), (1000, 2100, 384): (128, 128), (4096, 5120, 256): (256, 160), (4000, 5100, 384): (256, 160), (512, 24576, 256): (256, 192), (500, 24500, 384): (256, 192),
                     (768, 10880, 256): (256, 128), (4096, 7168, 7168): (256, 256), (4096, 2048, 7168): (128, 256), (1024, 4096, 7168): (128, 128),
                     (512, 4096, 2048): (64, 128), (257, 2112, 1024): (64, 64), (64, 7168, 2048): (64, 32), (64, 4096, 7168): (32, 32)}
# Plain FP8 calls the grouped and quantiser tests make on the side (first group through the plain entry, quantise-then-
# multiply): listed so that their kernels are compiled ahead of time as well.
FP8_SIDE_SHAPES = [(1024, 4096, 7168), (8192, 4096, 7168), (200, 384, 512), (1152, 512, 512), (128, 4096, 1024), (128, 320, 384),
                   (256, 200, 128), (256, 512, 512)]
# Problems the split-K plan covers on 256 compute units, with the (BLOCK_M, BLOCK_N, SPLIT_K) it makes (a CPU test keeps this
# true): every ring tile, every factor, ragged m and n, n that is no multiple of 8 (direct stores), K ranges of unequal
# length (49 k-tiles in 2 parts, 43 and 56 in 3).
FP8_SPLIT_K_PLAN_OF_SHAPE = {
    (17, 3076, 6272): (32, 32, 2), (33, 196, 5504): (32, 32, 3), (64, 196, 7168): (32, 32, 4), (31, 3588, 6272): (32, 32, 2),
    (33, 2112, 5376): (64, 32, 3), (50, 1536, 7168): (64, 32, 4), (64, 2112, 7168): (64, 32, 3),
    (100, 2112, 5376): (64, 64, 3), (65, 1536, 7168): (64, 64, 4),
    (200, 3076, 6144): (64, 128, 2), (100, 4100, 5376): (64, 128, 3), (129, 2112, 7168): (64, 128, 4),
    (300, 4100, 6144): (128, 128, 2), (200, 4100, 5376): (128, 128, 3), (129, 4096, 7168): (128, 128, 4),
    (64, 4096, 7168): (64, 64, 4), (128, 4096, 7168): (64, 128, 4), (5, 3076, 6144): (32, 32, 2), (1, 4096, 7168): (32, 32, 2),
}
# bf16 activations through the entry that chains the quantiser and the GEMM in one `launch`: a split-K plan, the weight-
# streaming kernel, unsplit tiles, rows that are no multiple of anything, and one whose codes do not fit the entry's scratch
# (two entry calls instead).
CAST_CHAIN_SHAPES = [(64, 4096, 7168), (1, 4096, 7168), (33, 2112, 5376), (7, 96, 640), (300, 2112, 1024), (512, 4096, 2048), (1100, 512, 4096)]
FP8_SPLIT_K_SHAPES = [s for s in FP8_SPLIT_K_PLAN_OF_SHAPE if s not in ((64, 4096, 7168), (128, 4096, 7168), (1, 4096, 7168))]
# The same for the dense GEMMs: the three tiles split-K plans use, every factor, ragged m and n, n that is no multiple of 8,
# k tails (3080 = 48 k-tiles and 8 elements, 7176), a dozen rows (where a plan goes before the weight-streaming kernel), six and
# eight parts.
DENSE_SPLIT_K_PLAN_OF_SHAPE = {
    (33, 196, 2048): (64, 64, 2), (100, 196, 3080): (64, 64, 3), (65, 196, 4096): (64, 64, 4),
    (129, 4100, 5632): (64, 128, 2), (200, 2112, 3072): (64, 128, 3), (129, 2112, 5120): (64, 128, 4),
    (300, 4100, 4096): (128, 128, 2), (200, 4100, 3080): (128, 128, 3), (200, 3076, 5120): (128, 128, 4),
    (64, 4096, 7168): (64, 64, 4), (256, 2048, 7168): (64, 128, 4), (12, 2052, 4096): (64, 64, 4),
    (20, 580, 7176): (64, 64, 6), (50, 1028, 16384): (64, 64, 8),
}
DENSE_SPLIT_K_SHAPES = list(DENSE_SPLIT_K_PLAN_OF_SHAPE)
# Grouped FP8 GEMMs: (rows per group, n, k, blocks of padding rows) and (groups, m_max, n, k, masked_m, expected_m).
# Long groups on 256-row tiles whose two 128-row halves belong to different groups, or one of them to padding: a padding
# block between the groups (negative entry) and one at the end; group 1 has 63 blocks, so it starts and the run ends on
# odd multiples of 128. The test also runs the rows rotated by one block, which moves every boundary by 128 rows.
GROUPED_TWO_PASS_CASE = ((8192, -128, 8064, 8192, 8192), 4096, 1024, 1)
# Sixteen groups of nine blocks: every other boundary falls in the middle of a 256-row tile, and the 73 tile rows are more
# than the 64 a wave looks at at once when it works out which rows hold two groups (those go first in the launch order).
GROUPED_TWO_GROUP_ROWS_FIRST_CASE = ((1152,) * 16, 512, 512, 1)
GROUPED_CONTIGUOUS_TEST_CASES = [
    GROUPED_TWO_PASS_CASE, GROUPED_TWO_GROUP_ROWS_FIRST_CASE,
    ((100, 128, 1, 300), 320, 384, 1), ((128, 128), 4096, 1024, 0), ((129,), 200, 128, 2),
    ((1024, 1024, 1024, 1024), 4096, 7168, 0), ((8192, 8192, 8192, 8192), 4096, 7168, 0),
    # long groups whose boundaries fall in the middle of 256-row tiles (two-pass tiles), with a trailing padding block
    ((1150, 900, 1300, 1100), 512, 512, 1),
    ((128, 128), 192, 256, 1),                       # the committed fixture
    # groups of a few hundred rows run the kernel that picks its tile height on the device: every boundary on a multiple of 256 rows
    # (it takes 256 x 256 tiles), every other one in the middle of such a tile (128 x 256 tiles)
    ((512,) * 16, 4096, 1024, 0), ((384, 640) * 8, 4096, 1024, 1),
]
# The same kernel built for small problems through explicit keys (the cost table gives those to smaller tiles): whole
# 256-row tiles, two groups in every other tile row, and a padding block in the middle with one boundary off.
GROUPED_ROWS_ON_DEVICE_CASES = [((512,) * 6, 768, 512, 0), ((384, 640) * 3, 768, 512, 1), ((512, 256, -128, 500, 512), 768, 384, 0)]
GROUPED_MASKED_TEST_CASES = [
    (3, 200, 320, 384, (200, 0, 77), 128), (4, 256, 4096, 1024, (1, 256, 130, 64), 64), (2, 64, 200, 128, (64, 3), 32),
    (4, 1024, 4096, 7168, (1024, 900, 512, 1), 1024),
    (2, 40, 192, 256, (40, 7), 40),                  # the committed fixture
    (2, 128, 512, 512, (128, 40), 128),              # the group of the graph-replay test
    # many groups, few rows of many: tile rows above expected_m exist in some groups, groups without rows, an odd group count
    (17, 384, 320, 384, (384, 0, 5, 64, 65, 0, 0, 200, 1, 384, 128, 129, 0, 7, 300, 64, 2), 64),
    (8, 1000, 512, 256, (0, 1000, 0, 0, 999, 130, 0, 1), 5000),      # a hint beyond m_max
]


# Shapes run under a compute-unit cap (set_num_sms): the 256 x 256 tiles (two rounds of 64 workgroups) and ring tiles.
NUM_SMS_CAP = 64
CAPPED_SHAPES = [(2048, 4096, 1024), (512, 4096, 2048), (300, 2112, 640)]


# A problem of 6 x 3 tiles of 256 x 256 (18: not a multiple of the 8 XCDs, so some XCDs' ranges end in an empty slot) run by
# 3 and 5 workgroups: walks that cross the XCDs' ranges. (m, n, k), caps.
ODD_CAP_CASE = ((1300, 768, 512), (3, 5))


def odd_cap_plans(cap: int):
    """((name, keys, arg_defs, includes, template) of the FP8 kernel, the same of the dense kernel) for ODD_CAP_CASE on
    256 x 256 tiles; the dense kernel takes its cap as a key, the FP8 kernel as a launch argument."""
    from yan_amd.jit_kernels import bf16_gemm, gemm
    (m, n, k), _ = ODD_CAP_CASE
    name, keys, arg_defs, code_template = fp8_explicit_tile_plan(256, 256, n, k)
    dense_keys = {'BLOCK_M': 256, 'BLOCK_N': 256, 'NUM_STAGES': 2, 'NUM_SMS': cap}
    return ((name, keys, arg_defs, gemm.includes, code_template),
            ('gemm_bf16_tn', dense_keys, bf16_gemm._arg_defs(torch.bfloat16), bf16_gemm.includes, bf16_gemm.template))


# Shapes run with empirical tile selection (YAN_TUNE_TILES=1): three candidate tiles each, for both GEMMs.
TUNED_SHAPES = [(4096, 5120, 5120), (2048, 7168, 7168)]


# FP8 tiles the cost model does not offer but the kernel supports, built through explicit keys: their wave slabs are
# 112, 96 and 80 columns wide, which straddle the 128-wide weight-scale blocks (two scale products per k-tile and a select
# per row of atoms) and do not divide the 64 lanes of the staged epilogue's row stores. (BLOCK_M, BLOCK_N, (m, n, k)).
FP8_EXPLICIT_TILE_CASES = [(256, 224, (600, 1344, 640)), (256, 224, (300, 1000, 384)), (256, 192, (520, 1156, 512)),
                           (64, 160, (1000, 2100, 384)), (64, 160, (200, 1156, 1024))]


def fp8_explicit_tile_plan(block_m: int, block_n: int, n: int, k: int):
    """(name, keys, arg_defs, template) of the FP8 JIT kernel with this tile and token-contiguous scales."""
    from yan_amd.jit_kernels import gemm
    from yan_amd.jit_kernels.heuristics import get_fp8_num_stages
    keys = {'N': n, 'K': k, 'BLOCK_M': block_m, 'BLOCK_N': block_n, 'NUM_STAGES': get_fp8_num_stages(block_m, block_n),
            'NUM_TMA_MULTICAST': 1}
    return 'gemm_fp8_fp8_bf16_nt', keys, gemm.arg_defs, gemm.template


def grouped_rows_on_device_plan(num_groups: int, n: int, k: int):
    """(name, keys, arg_defs, template) of the contiguous grouped kernel that picks its tile height on the device, whatever the
    cost table would give the problem."""
    from yan_amd.jit_kernels import m_grouped_gemm
    keys = {'N': n, 'K': k, 'BLOCK_M': 256, 'BLOCK_N': 256, 'NUM_GROUPS': num_groups, 'NUM_STAGES': 2, 'NUM_TMA_MULTICAST': 1,
            'GEMM_TYPE': 'GroupedContiguous', 'ROWS': 'picked on the device'}
    return 'm_grouped_gemm_fp8_fp8_bf16_nt_rows_on_device', keys, m_grouped_gemm.arg_defs, m_grouped_gemm.rows_on_device_template


def jit_kernels_in_use(num_cus: int = 256):
    """(name, arg_defs, code) of every distinct JIT kernel the shapes above, and the quantisers select."""
    from yan_amd.jit import cpp_format, generate
    from yan_amd.jit_kernels import bf16_gemm, fp8_cast, gemm, m_grouped_gemm, simple_gemm
    kernels = {}

    def add(name, arg_defs, includes, code_template, keys):
        code = generate(includes, arg_defs, cpp_format(code_template, keys))
        kernels.setdefault((name, code), (name, arg_defs, code))

    # the last four: shapes only the benchmark's --also legs run
    for m, n, k in DENSE_TEST_SHAPES + REFERENCE_DENSE_TEST_SHAPES + DENSE_SPLIT_K_SHAPES + [(256, 512, 512), (4096, 5120, 5120), (2048, 7168, 7168), (4096, 7168, 16384), (8192, 8192, 9216)]:
        for dtype in (torch.bfloat16, torch.half):
            if m and n:
                name, keys, arg_defs = bf16_gemm.dense_kernel_plan(m, n, k, dtype, num_cus)
                add(name, arg_defs, bf16_gemm.includes, bf16_gemm.template, keys)
                split = bf16_gemm.dense_split_k_plan(m, n, k, dtype, num_cus)
                if split is not None:
                    name, keys, arg_defs = split
                    add(name, arg_defs, bf16_gemm.includes, bf16_gemm.split_k_template, keys)
    for dtype in (torch.bfloat16, torch.half):
        for m, n, k in DENSE_BOTH_KERNELS_SHAPES:
            name, keys, arg_defs = bf16_gemm.dense_kernel_plan(m, n, k, dtype, num_cus)
            assert keys['BLOCK_M'] == 256 and keys['BLOCK_N'] >= 160, (m, n, k)
            add(name, arg_defs, bf16_gemm.includes, bf16_gemm.template, keys)
            for cap in (7, 100):
                name, capped_keys, arg_defs = bf16_gemm.dense_kernel_plan(m, n, k, dtype, num_cus, cap)
                add(name, arg_defs, bf16_gemm.includes, bf16_gemm.template, capped_keys)
            name, keys, arg_defs, code_template = dense_explicit_plan((keys['BLOCK_M'], keys['BLOCK_N']), dtype, eight_waves=True)
            add(name, arg_defs, bf16_gemm.includes, code_template, keys)
    for block_n in (160, 192, 224, 256):           # every width with the tile given, on either kernel (DENSE_SEEDED_BOTH_KERNELS_SHAPES)
        for eight_waves in (False, True):
            name, keys, arg_defs, code_template = dense_explicit_plan((256, block_n), torch.bfloat16, eight_waves)
            add(name, arg_defs, bf16_gemm.includes, code_template, keys)
    for m, n, k in REFERENCE_FLOAT_TEST_SHAPES + FLOAT_TEST_SHAPES + [(5120, 2048, 4096)]:
        name, keys, arg_defs = simple_gemm.float_kernel_plan(m, n, num_cus)
        add(name, arg_defs, simple_gemm.includes, simple_gemm.template, keys)
    for m, n, k in FP8_TEST_SHAPES + FP8_SIDE_SHAPES + FP8_SPLIT_K_SHAPES:
        for token_contiguous in (True, False) if m else ():     # both layouts of the activation scales
            name, keys, arg_defs, _, code_template = gemm.fp8_kernel_plan(m, n, k, num_cus, token_contiguous)
            add(name, arg_defs, gemm.includes, code_template, keys)
            split = gemm.fp8_split_k_plan(m, n, k, num_cus, token_contiguous)
            if split is not None:
                name, keys, arg_defs, code_template = split
                add(name, arg_defs, gemm.includes, code_template, keys)
    for m, n, k in CAST_CHAIN_SHAPES:
        chain = gemm.fp8_cast_chain_plan(m, n, k, num_cus)
        if chain is not None:
            name, keys, arg_defs, code_template, _ = chain
            add(name, arg_defs, gemm.cast_includes, code_template, keys)
        # what two entry calls run for the same sizes
        name, keys, arg_defs, _, code_template = gemm.fp8_kernel_plan(m, n, k, num_cus, True)
        add(name, arg_defs, gemm.includes, code_template, keys)
        split = gemm.fp8_split_k_plan(m, n, k, num_cus, True)
        if split is not None:
            name, keys, arg_defs, code_template = split
            add(name, arg_defs, gemm.includes, code_template, keys)
    for m, n, k in CAPPED_SHAPES:
        for cus, cap in ((num_cus, 0), (num_cus, NUM_SMS_CAP), (NUM_SMS_CAP, NUM_SMS_CAP)):
            name, keys, arg_defs = bf16_gemm.dense_kernel_plan(m, n, k, torch.bfloat16, cus, cap)
            add(name, arg_defs, bf16_gemm.includes, bf16_gemm.template, keys)
        for cus in (num_cus, NUM_SMS_CAP):
            for token_contiguous in (False, True):      # row-major scales of a large problem reach the kernel token-contiguous
                name, keys, arg_defs, _, code_template = gemm.fp8_kernel_plan(m, n, k, cus, token_contiguous)
                add(name, arg_defs, gemm.includes, code_template, keys)
    for block_m, block_n, (m, n, k) in FP8_EXPLICIT_TILE_CASES:
        name, keys, arg_defs, code_template = fp8_explicit_tile_plan(block_m, block_n, n, k)
        add(name, arg_defs, gemm.includes, code_template, keys)
        name, keys, arg_defs, _, code_template = gemm.fp8_kernel_plan(m, n, k, num_cus, True)
        add(name, arg_defs, gemm.includes, code_template, keys)
    for cap in (0,) + ODD_CAP_CASE[1]:
        for name, keys, arg_defs, includes, code_template in odd_cap_plans(cap):
            add(name, arg_defs, includes, code_template, keys)
    for m, n, k in TUNED_SHAPES:
        name, keys, space, arg_defs = bf16_gemm.dense_tuning_plan(m, n, k, torch.bfloat16, num_cus)
        for extra in space:
            add(name, arg_defs, bf16_gemm.includes, bf16_gemm.template, {**keys, **extra})
        name, keys, space, arg_defs, code_template = gemm.fp8_tuning_plan(m, n, k, num_cus, True)
        for extra in space:
            add(name, arg_defs, gemm.includes, code_template, {**keys, **extra})
    for kind in ('per_token', 'per_block'):
        for dtype in (torch.bfloat16, torch.float32):
            name, keys, arg_defs, code_template = fp8_cast.cast_kernel_plan(kind, dtype)
            add(name, arg_defs, fp8_cast.includes, code_template, keys)
    for rows, n, k, pad_blocks in GROUPED_CONTIGUOUS_TEST_CASES:
        m = sum((abs(r) + 127) // 128 * 128 for r in rows) + 128 * pad_blocks
        name, keys, arg_defs, _ = m_grouped_gemm.grouped_kernel_plan('GroupedContiguous', sum(1 for r in rows if r > 0), m, n, k, num_cus)
        add(name, arg_defs, m_grouped_gemm.includes, m_grouped_gemm.rows_on_device_template if 'ROWS' in keys else m_grouped_gemm.template, keys)
    for groups, m_max, n, k, _, expected_m in GROUPED_MASKED_TEST_CASES:
        name, keys, arg_defs, _ = m_grouped_gemm.grouped_kernel_plan('GroupedMasked', groups, min(expected_m, m_max), n, k, num_cus)
        add(name, arg_defs, m_grouped_gemm.includes, m_grouped_gemm.template, keys)
    # contiguous layouts only the benchmark's --also legs run
    for rows, n, k in (((896, 1152) * 4, 4096, 7168), ((1024,) * 8, 4096, 7168), ((512,) * 16, 4096, 7168), ((384, 640) * 8, 4096, 7168)):
        name, keys, arg_defs, _ = m_grouped_gemm.grouped_kernel_plan('GroupedContiguous', len(rows), sum(rows), n, k, num_cus)
        add(name, arg_defs, m_grouped_gemm.includes, m_grouped_gemm.rows_on_device_template if 'ROWS' in keys else m_grouped_gemm.template, keys)
    for rows, n, k, _ in GROUPED_ROWS_ON_DEVICE_CASES:
        name, keys, arg_defs, code_template = grouped_rows_on_device_plan(sum(1 for r in rows if r > 0), n, k)
        add(name, arg_defs, m_grouped_gemm.includes, code_template, keys)
    # the grouped layouts under the compute-unit cap: tiles chosen for NUM_SMS_CAP units
    rows, n, k, pad_blocks = GROUPED_TWO_GROUP_ROWS_FIRST_CASE
    name, keys, arg_defs, _ = m_grouped_gemm.grouped_kernel_plan('GroupedContiguous', len(rows), sum(rows) + 128 * pad_blocks, n, k, NUM_SMS_CAP)
    add(name, arg_defs, m_grouped_gemm.includes, m_grouped_gemm.rows_on_device_template if 'ROWS' in keys else m_grouped_gemm.template, keys)
    groups, m_max, n, k, _, expected_m = GROUPED_MASKED_TEST_CASES[6]
    name, keys, arg_defs, _ = m_grouped_gemm.grouped_kernel_plan('GroupedMasked', groups, min(expected_m, m_max), n, k, NUM_SMS_CAP)
    add(name, arg_defs, m_grouped_gemm.includes, m_grouped_gemm.template, keys)
    return list(kernels.values())


def prebuild_jit_kernels(num_cus: int = 256, verbose: bool = False, jobs: int = 0) -> int:
    """Compile every JIT kernel of `jit_kernels_in_use` (hipcc cross-compiles for gfx950 without a GPU) into the
    current kernel cache, `jobs` compilers at a time (default: one per CPU, at most 8). Returns the number of kernels."""
    import os
    from concurrent.futures import ThreadPoolExecutor
    from yan_amd.jit import build
    kernels = jit_kernels_in_use(num_cus)
    jobs = jobs or max(1, min(8, os.cpu_count() or 1))

    def one(kernel):
        runtime = build(*kernel)
        if verbose:
            print(f'built {kernel[0]} -> {runtime.path}')
        return runtime

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(one, kernels))
    return len(kernels)
