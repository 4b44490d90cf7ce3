"""Host-side logic that needs no device: helpers, tile heuristics, tuner selection rules, entry-point argument
checks (reference: yan/jit_kernels/utils.py:32-85, yan/jit_kernels/tuner.py:12-78, yan/jit_kernels/cute_gemm.py:21-30)."""
import os

import pytest
import torch

import yan_amd as yan
from yan_amd.jit_kernels import heuristics, tuner as tuner_mod, bf16_gemm, gemm, simple_gemm


def test_ceil_div_and_alignment():
    assert yan.ceil_div(7, 2) == 4 and yan.ceil_div(8, 2) == 4 and yan.ceil_div(0, 128) == 0 and yan.ceil_div(1, 128) == 1
    assert yan.get_m_alignment_for_contiguous_layout() == 128


def test_get_col_major_tensor():
    x = torch.arange(12, dtype=torch.float32).view(3, 4)
    y = yan.get_col_major_tensor(x)
    assert y.shape == x.shape and torch.equal(x, y) and y.stride() == (1, 3)
    assert yan.get_col_major_tensor(y).data_ptr() == y.data_ptr()          # already token-contiguous: untouched
    b = torch.arange(24, dtype=torch.float32).view(2, 3, 4)
    yb = yan.get_col_major_tensor(b)
    assert torch.equal(b, yb) and yb.stride(1) == 1 and yb.stride(2) == 3
    with pytest.raises(AssertionError):
        yan.get_col_major_tensor(torch.zeros(3))


def test_tile_heuristics_fill_256_cus():
    # the headline FP8 shape: 256x256 tiles give 448 workgroups = 1.75 rounds
    assert heuristics.get_best_fp8_config(4096, 7168, 7168, 256) in ((256, 256), (256, 128), (128, 256))
    assert heuristics.get_best_dense_config(8192, 8192, 8192, 256) == (256, 256)
    # a skinny problem must not pick a tile that leaves most CUs idle
    bm, bn = heuristics.get_best_fp8_config(64, 4096, 7168, 256)
    assert yan.ceil_div(64, bm) * yan.ceil_div(4096, bn) >= 128
    # ... the decode shape runs the tiled kernel on 32 x 32 tiles (the 256 tiles of least operand traffic) with a deep ring of LDS stages, and up to 16 rows go
    # to the weight-streaming kernel (one workgroup per 16 weight rows) while those workgroups fit the chip at once
    assert heuristics.get_fp8_tile(64, 4096, 7168, 256) == (32, 32) and heuristics.get_fp8_num_stages(32, 32) == 12
    assert heuristics.get_fp8_tile(1, 4096, 7168, 256) == (16, 16) and heuristics.get_fp8_tile(16, 2048, 7168, 256) == (16, 16)
    assert heuristics.get_skinny_fp8_config(17, 4096, 7168, 256) == 0 and heuristics.get_skinny_fp8_config(16, 7168, 7168, 256) == 0
    assert heuristics.get_fp8_num_stages(256, 256) == 2 and heuristics.get_dense_num_stages(256, 256) == 2
    assert heuristics.get_dense_num_stages(64, 64) == 8 and heuristics.get_dense_num_stages(128, 256) == 3
    # tiny problems get the smallest tile
    assert heuristics.get_best_dense_config(64, 64, 64, 256) == (64, 64)
    # fp32: full tiles for large problems, K-split tiles (below 128 rows) when a 128-row tiling leaves CUs idle
    assert heuristics.get_best_float_config(8192, 8192, 256) == (256, 256)
    assert heuristics.get_best_float_config(4096, 7168, 256) == (128, 128)          # 1792 tiles: exactly 7 rounds
    assert heuristics.get_best_float_config(128, 2112, 256) == (32, 64)             # 33 tiles of 128 x 64 would use 33 CUs
    assert heuristics.get_best_float_config(128, 64, 256) == (32, 32)
    ranked = heuristics.rank_tiles(4096, 7168, 256, heuristics._FP8_TILES)
    assert ranked == sorted(ranked) and len(ranked) == len(heuristics._FP8_TILES)


def test_activation_scales_are_relaid_only_where_it_pays():
    """Large problems get token-contiguous activation scales (same values), small ones and scales that already are
    token-contiguous pass through untouched."""
    from yan_amd.jit_kernels.utils import scales_for_kernel, SCALE_RELAYOUT_MIN_FLOP
    rows = torch.arange(512 * 56, dtype=torch.float32).reshape(512, 56)
    assert scales_for_kernel(rows, SCALE_RELAYOUT_MIN_FLOP / 2) is rows
    big = scales_for_kernel(rows, SCALE_RELAYOUT_MIN_FLOP)
    assert big.stride() == (1, 512) and torch.equal(big, rows)
    assert scales_for_kernel(big, 1e15) is big
    one_block = rows[:, :1]
    assert scales_for_kernel(one_block, 1e15) is one_block
    batched = torch.arange(3 * 64 * 8, dtype=torch.float32).reshape(3, 64, 8)
    relaid = scales_for_kernel(batched, 1e15)
    assert relaid.stride() == (64 * 8, 1, 64) and torch.equal(relaid, batched)
    assert scales_for_kernel(relaid, 1e15) is relaid


def test_split_k_plans():
    """K is split when the unsplit tiles leave the chip short of work and K is long; every plan fits one round of
    workgroups and the workspace, leaves each part 14 k-tiles or more (24 of two), and the shapes of the GPU suite get the plans the
    suite expects (every ring tile, every factor)."""
    import harness
    plan = heuristics.get_split_k_fp8_config
    assert plan(64, 4096, 7168, 256) == (64, 64, 4) and plan(32, 2112, 7168, 256) == (32, 32, 3)
    assert plan(256, 7168, 7168, 256) == (128, 128, 2) and plan(128, 7168, 16384, 256) == (128, 128, 4)
    # short K, a weight matrix that takes as long to stream as to multiply, work for every compute unit, few rows
    assert plan(64, 7168, 2048, 256) is None and plan(64, 16384, 7168, 256) is None and plan(4096, 7168, 7168, 256) is None
    assert plan(16, 4096, 2048, 256) is None and plan(0, 4096, 7168, 256) is None
    assert plan(16, 4096, 7168, 256) == (32, 32, 2) and plan(1, 2112, 7168, 256) == (32, 32, 3)      # before the weight-streaming kernel
    for shape, expected in harness.FP8_SPLIT_K_PLAN_OF_SHAPE.items():
        assert plan(*shape, 256) == expected, shape
    assert {(bm, bn) for bm, bn, _ in harness.FP8_SPLIT_K_PLAN_OF_SHAPE.values()} == set(heuristics._FP8_SPLIT_K_TILE_US)
    assert {s for _, _, s in harness.FP8_SPLIT_K_PLAN_OF_SHAPE.values()} == set(heuristics.FP8_SPLIT_K_FACTORS)
    for m in (17, 33, 64, 100, 129, 256, 300, 512, 1024):
        for n in (196, 1536, 2112, 4096, 4100, 7168, 24576):
            for k in (1536, 3072, 3200, 4608, 7168, 16384):
                for cus in (256, 64, 8):
                    p = plan(m, n, k, cus)
                    if p is None:
                        continue
                    bm, bn, split = p
                    slots = yan.ceil_div(yan.ceil_div(m, bm) * yan.ceil_div(n, bn), 8) * 8
                    assert slots * split <= cus and yan.ceil_div(k // 128, split) >= (24 if split == 2 else 14)
                    assert gemm.SPLIT_K_COUNTER_BYTES + slots * split * bm * bn * 4 <= gemm.SPLIT_K_WORKSPACE_BYTES
                    assert slots * 8 * 4 <= gemm.SPLIT_K_COUNTER_BYTES
                    assert heuristics.get_fp8_num_stages(bm, bn) > 2          # a ring tile
    name, keys, defs, tmpl = gemm.fp8_split_k_plan(64, 4096, 7168, 256)
    assert name == 'gemm_fp8_fp8_bf16_nt_split_k' and keys['SPLIT_K'] == 4 and defs[-2:] == (('workspace', torch.uint8), ('workspace_bytes', int))
    assert 'run_split_k<4>' in yan.jit.cpp_format(tmpl, keys)
    strided = gemm.fp8_split_k_plan(64, 4096, 7168, 256, False)
    assert strided[0].endswith('_strided') and strided[2][-2:] == (('lhs_scales_stride_m', int), ('lhs_scales_stride_k', int))
    assert gemm.fp8_split_k_plan(4096, 7168, 7168, 256) is None


def test_dense_split_k_plans():
    """The dense GEMMs split K by the same rule with their own tile numbers: plans fit one round and the workspace, leave each
    part 16 k-tiles or more, and the shapes of the GPU suite get the plans the suite expects."""
    import harness
    plan = heuristics.get_split_k_dense_config
    assert plan(64, 4096, 7168, 256) == (64, 64, 4) and plan(256, 7168, 16384, 256) == (128, 128, 2)
    assert plan(256, 7168, 2048, 256) is None and plan(256, 24576, 1536, 256) is None and plan(8192, 8192, 8192, 256) is None
    assert plan(7, 4096, 7168, 256) is None and plan(16, 4096, 16384, 256) is None          # the one-atom weight-streaming kernel's
    assert plan(8, 4096, 7168, 256) == (64, 64, 4) and plan(17, 4096, 16384, 256) == (64, 64, 4)
    for shape, expected in harness.DENSE_SPLIT_K_PLAN_OF_SHAPE.items():
        assert plan(*shape, 256) == expected, shape
    assert {(bm, bn) for bm, bn, _ in harness.DENSE_SPLIT_K_PLAN_OF_SHAPE.values()} == set(heuristics._DENSE_SPLIT_K_EXTRA_US)
    assert {s for _, _, s in harness.DENSE_SPLIT_K_PLAN_OF_SHAPE.values()} == set(heuristics.DENSE_SPLIT_K_FACTORS)
    assert all((bm, bn) == (64, 64) for bm, bn, s in harness.DENSE_SPLIT_K_PLAN_OF_SHAPE.values() if s > 4)
    assert set(heuristics._DENSE_SPLIT_K_TILE_US) == {t for t in heuristics._DENSE_TILES if heuristics.get_dense_num_stages(*t) > 2}
    for m in (33, 64, 100, 129, 256, 300, 512, 1024):
        for n in (196, 1536, 2112, 4096, 4100, 7168, 24576):
            for k in (1536, 2048, 3080, 4608, 7168, 16384):
                for cus in (256, 64, 8):
                    p = plan(m, n, k, cus)
                    if p is None:
                        continue
                    bm, bn, split = p
                    slots = yan.ceil_div(yan.ceil_div(m, bm) * yan.ceil_div(n, bn), 8) * 8
                    assert slots * split <= cus and yan.ceil_div(yan.ceil_div(k, 64), split) >= 16
                    assert gemm.SPLIT_K_COUNTER_BYTES + slots * split * bm * bn * 4 <= gemm.SPLIT_K_WORKSPACE_BYTES
                    assert slots * 4 * 4 <= gemm.SPLIT_K_COUNTER_BYTES
    name, keys, defs = bf16_gemm.dense_split_k_plan(64, 4096, 7168, torch.half, 256)
    assert name == 'gemm_fp16_tn_split_k' and keys['SPLIT_K'] == 4 and defs[-2:] == (('workspace', torch.uint8), ('workspace_bytes', int))
    assert 'gemm_tn_split_k<BLOCK_M, BLOCK_N, kNumStages, kSplitK>' in bf16_gemm.split_k_template
    assert bf16_gemm.dense_split_k_plan(8192, 8192, 8192, torch.bfloat16, 256) is None


def test_fp8_shapes_of_the_gpu_suite_reach_every_tile_of_the_cost_table():
    import harness
    for shape, tile in harness.FP8_TILE_OF_SHAPE.items():
        assert shape in harness.FP8_TEST_SHAPES + harness.FP8_SIDE_SHAPES
        assert heuristics.get_fp8_tile(*shape, 256) == tile, shape
    assert set(harness.FP8_TILE_OF_SHAPE.values()) == set(heuristics._FP8_TILES)
    # two full rounds of 256 x 160 tiles beat 1.25 rounds of 256 x 256 tiles
    assert heuristics.get_best_fp8_config(4096, 5120, 5120, 256) == (256, 160)
    # the grouped layouts keep to widths of 64, 128 and 256
    assert heuristics.get_best_grouped_fp8_config(4096, 5120, 5120, 256, 1, 128, 4)[1] in (64, 128, 256)


def test_dense_shapes_of_the_gpu_suite_reach_every_tile_of_the_8_wave_kernel():
    """A change of the cost table must not silently take the 256 x {160, 192, 224} tiles, or the 192-wide ring tiles, out of the
    parity tests."""
    import harness
    for shape, tile in harness.DENSE_TILE_OF_SHAPE.items():
        assert shape in harness.DENSE_TEST_SHAPES
        assert heuristics.get_dense_tile(*shape, 256) == tile, shape
        if tile[1] != 16:
            assert heuristics.get_dense_num_stages(*tile) == (2 if tile[0] == 256 else {(128, 192): 4, (64, 192): 5}[tile])
    assert {t for t in harness.DENSE_TILE_OF_SHAPE.values()} == {(256, 160), (256, 192), (256, 224), (256, 256), (128, 192), (64, 192),
                                                                 (16, 16), (32, 16)}
    # shapes on which the launcher of the 256-row tiles takes the 4-wave kernel, every width among them, and shapes on which
    # it cannot
    for m, n, k in harness.DENSE_BOTH_KERNELS_SHAPES + [(8192, 8192, 8192)]:
        tile = heuristics.get_dense_tile(m, n, k, 256)
        assert tile[0] == 256 and tile[1] >= 160 and k % 64 == 0 and k >= 256 and n % 8 == 0
    assert {heuristics.get_dense_tile(*shape, 256)[1] for shape in harness.DENSE_BOTH_KERNELS_SHAPES} == {160, 192, 224, 256}
    assert 1000 % 64 != 0 and 5004 % 8 != 0 and 520 % 64 != 0 and 264 % 64 != 0 and 72 < 256
    # the weight-streaming kernel: one round of workgroups, whole K blocks, two atoms only on long K
    assert heuristics.get_skinny_dense_config(16, 4096, 7168, 256) == 1 and heuristics.get_skinny_dense_config(16, 4112, 7168, 256) == 0
    assert heuristics.get_skinny_dense_config(16, 4096, 7176, 256) == 0 and heuristics.get_skinny_dense_config(33, 4096, 7168, 256) == 0
    assert heuristics.get_skinny_dense_config(32, 4096, 1024, 256) == 0 and heuristics.get_skinny_dense_config(32, 4096, 2048, 256) == 2
    assert heuristics.get_skinny_dense_config(16, 1024, 7168, 64) == 1 and heuristics.get_skinny_dense_config(16, 2048, 7168, 64) == 0


def test_kernel_plans_keep_reference_keys_and_argument_order():
    name, keys, defs = bf16_gemm.dense_kernel_plan(4096, 7168, 2048, torch.bfloat16, 256)
    assert name == 'gemm_bf16_tn' and sorted(keys) == ['BLOCK_M', 'BLOCK_N', 'NUM_SMS', 'NUM_STAGES'] and keys['NUM_SMS'] == 0
    assert bf16_gemm.dense_kernel_plan(4096, 7168, 2048, torch.bfloat16, 64, 64)[1]['NUM_SMS'] == 64
    assert [d[0] for d in defs] == ['m', 'n', 'k', 'A', 'B', 'C', 'stream']
    assert bf16_gemm.dense_kernel_plan(4096, 7168, 2048, torch.half, 256)[0] == 'gemm_fp16_tn'
    name, keys, defs, smem, _ = gemm.fp8_kernel_plan(4096, 7168, 7168, 256)
    assert name == 'gemm_fp8_fp8_bf16_nt'
    assert sorted(keys) == ['BLOCK_M', 'BLOCK_N', 'K', 'N', 'NUM_STAGES', 'NUM_TMA_MULTICAST']
    # the reference's nine run-time names, exactly (yan/jit_kernels/gemm.py:23-30), for token-contiguous activation scales
    assert [d[0] for d in defs] == ['lhs', 'lhs_scales', 'rhs', 'rhs_scales', 'out', 'm', 'stream', 'num_sms', 'smem_size']
    assert defs is gemm.arg_defs and gemm.fp8_kernel_plan(4096, 7168, 7168, 256)[4] is gemm.template
    # any other strided layout: the same, plus the two strides
    strided = gemm.fp8_kernel_plan(4096, 7168, 7168, 256, False)
    assert [d[0] for d in strided[2]] == [d[0] for d in defs] + ['lhs_scales_stride_m', 'lhs_scales_stride_k'] and strided[1] == keys
    assert strided[0] == 'gemm_fp8_fp8_bf16_nt_strided'           # its own name: the tuner memoises per (name, keys)
    name, fkeys, defs = simple_gemm.float_kernel_plan(4096, 7168, 256)
    assert name == 'gemm_float_nt' and sorted(fkeys) == ['BLOCK_M', 'BLOCK_N']
    assert [d[0] for d in defs] == ['m', 'n', 'k', 'alpha', 'A', 'ldA', 'B', 'ldB', 'beta', 'C', 'ldC', 'stream']
    assert keys['N'] == 7168 and keys['K'] == 7168 and smem == 2 * (keys['BLOCK_M'] + keys['BLOCK_N']) * 128 <= 160 * 1024


def test_entry_points_reject_bad_arguments_before_touching_a_device():
    a, b = torch.zeros(8, 16, dtype=torch.bfloat16), torch.zeros(4, 16, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        yan.gemm_bf16_tn(a, b, torch.zeros(8, 8, dtype=torch.bfloat16))          # n mismatch
    with pytest.raises(AssertionError):
        yan.gemm_bf16_tn(a.half(), b, torch.zeros(8, 4, dtype=torch.bfloat16))   # dtype mismatch
    with pytest.raises(AssertionError):
        yan.gemm_fp16_tn(a, b, torch.zeros(8, 4, dtype=torch.bfloat16))
    # empty problems return before any device call
    yan.gemm_bf16_tn(torch.zeros(0, 16, dtype=torch.bfloat16), b, torch.zeros(0, 4, dtype=torch.bfloat16))
    yan.gemm_fp16_tn(torch.zeros(8, 16, dtype=torch.half), torch.zeros(0, 16, dtype=torch.half), torch.zeros(8, 0, dtype=torch.half))
    # fp32 GEMM (yan/jit_kernels/simple_gemm.py:25-32): m % 128, n % 64, dtypes, shapes; operands M- / N-contiguous
    x, y = yan.get_col_major_tensor(torch.zeros(128, 16)), yan.get_col_major_tensor(torch.zeros(64, 16))
    with pytest.raises(AssertionError):
        yan.gemm_float_nt(x[:100], y, torch.zeros(100, 64))
    with pytest.raises(AssertionError):
        yan.gemm_float_nt(x, y[:32], torch.zeros(128, 32))
    with pytest.raises(AssertionError):
        yan.gemm_float_nt(x, y, torch.zeros(128, 128))
    with pytest.raises(AssertionError):
        yan.gemm_float_nt(x.double(), y, torch.zeros(128, 64))
    with pytest.raises(AssertionError):     # row-major operands would be read as their transposes
        yan.gemm_float_nt(torch.zeros(128, 16), y, torch.zeros(128, 64))
    yan.gemm_float_nt(yan.get_col_major_tensor(torch.zeros(0, 16)), y, torch.zeros(0, 64))
    q = torch.zeros(0, 128, dtype=torch.float8_e4m3fn)
    w = torch.zeros(128, 128, dtype=torch.float8_e4m3fn)
    yan.gemm_fp8_fp8_bf16_nt((q, torch.zeros(0, 1)), (w, torch.ones(1, 1)), torch.zeros(0, 128, dtype=torch.bfloat16))
    with pytest.raises(AssertionError):     # k not a multiple of the 128-deep scale block
        yan.gemm_fp8_fp8_bf16_nt((torch.zeros(4, 64, dtype=torch.float8_e4m3fn), torch.zeros(4, 1)),
                                 (torch.zeros(128, 64, dtype=torch.float8_e4m3fn), torch.ones(1, 1)),
                                 torch.zeros(4, 128, dtype=torch.bfloat16))
    with pytest.raises(AssertionError):     # wrong scale-table shape
        yan.gemm_fp8_fp8_bf16_nt((torch.zeros(4, 128, dtype=torch.float8_e4m3fn), torch.zeros(4, 2)),
                                 (w, torch.ones(1, 1)), torch.zeros(4, 128, dtype=torch.bfloat16))


class _FakeRuntime:
    def __init__(self, tag, rc=0):
        self.tag, self.rc, self.calls = tag, rc, 0

    def __call__(self, *args):
        self.calls += 1
        return self.rc


def test_tuner_memoises_skips_illegal_and_keeps_the_fastest(monkeypatch):
    built = []
    times = {'a': 3.0, 'b': 1.0, 'c': 2.0, 'bad': 0.1}

    def fake_build(name, arg_defs, code):
        tag = code.split('TAG=')[1].split(';')[0]
        rt = _FakeRuntime(tag, rc=5 if tag == 'bad' else 0)
        built.append(rt)
        return rt

    monkeypatch.setattr(tuner_mod, 'build', fake_build)
    monkeypatch.setattr(tuner_mod, '_time_candidate', lambda rt, args: times[rt.tag])
    t = tuner_mod.JITTuner()
    kw = dict(includes=(), arg_defs=(('n', int),), template='\nint TAG={T}; int k={KEY};\n', args=(1,))
    space = ({'T': 'a'}, {'T': 'bad'}, {'T': 'b'}, {'T': 'c'})
    best = t.compile_and_tune(name='op', keys={'KEY': 1}, space=space, **kw)
    assert best.tag == 'b' and len(built) == 4
    assert [r.calls for r in built] == [1, 1, 1, 1]              # one validity run each; the illegal one is not timed
    # memo hit: same name and keys (in any order) -> no new build
    assert t.compile_and_tune(name='op', keys={'KEY': 1}, space=space, **kw) is best and len(built) == 4
    # different keys -> new entry; empty space -> exactly one build, not run, time 0
    one = t.compile_and_tune(name='op', keys={'KEY': 2, 'T': 'c'}, space=(), **kw)
    assert one.tag == 'c' and one.calls == 0 and len(built) == 5
    # every candidate illegal -> assertion
    with pytest.raises(AssertionError, match='Failed to tune'):
        t.compile_and_tune(name='op2', keys={'KEY': 3}, space=({'T': 'bad'}, {'T': 'bad'}), **kw)


def test_reference_package_name_is_an_alias():
    """Code written against the reference imports `yan` (tests/test_cute.py:5-6 there); here that name resolves to
    this package, with the names that test uses."""
    import yan as by_reference_name
    assert by_reference_name is yan
    for name in ('gemm_fp16_tn', 'bench_kineto', 'get_col_major_tensor', 'calc_diff', 'jit', 'jit_kernels', 'gemm'):
        assert hasattr(by_reference_name, name), name
    assert callable(by_reference_name.jit_kernels.cute_gemm_accuracy_test)


def test_tile_scheduler_visits_every_tile_once_and_walks_cover_every_slot(tmp_path, repo_root):
    """XcdTileScheduler::tile_of and capped_grid are __host__ __device__: the checks live in tests/scheduler_host.cpp,
    compiled for the host only."""
    import subprocess
    from yan_amd.jit.compiler import get_hipcc_compiler, get_jit_include_dir
    exe = tmp_path / 'scheduler_host'
    subprocess.check_call([get_hipcc_compiler()[0], '-x', 'hip', '--cuda-host-only', '-std=c++20', '-O1', f'-I{get_jit_include_dir()}',
                           os.path.join(repo_root, 'tests', 'scheduler_host.cpp'), '-o', str(exe)])
    done = subprocess.run([str(exe)], stdout=subprocess.PIPE, universal_newlines=True)
    assert done.returncode == 0 and done.stdout.startswith('ok '), done.stdout
    assert int(done.stdout.split()[1]) > 400


@pytest.mark.parametrize('shape,dtype_name', [((8192, 8192, 8192), 'bfloat16'), ((4096, 5120, 5120), 'bfloat16'), ((8192, 8192, 8192), 'half')])
def test_tied_accumulators_of_the_8_wave_kernel_stay_where_the_mfmas_left_them(tmp_path, shape, dtype_name):
    """The 8-wave dense kernel writes its MFMAs as asm statements whose destination is their own addend. The compiler does
    not know how long such an instruction takes, so nothing but MFMAs may touch an accumulator register between the first
    and the last MFMA of the main loop (a compiler-made copy right behind an MFMA would read a sum that is not there yet),
    and what reads them first afterwards must sit behind the wait states written in the source. Checked on the generated
    code: compiled for the device only, no GPU needed."""
    import re
    import subprocess
    from yan_amd.jit import cpp_format, generate
    from yan_amd.jit.compiler import get_hipcc_compiler, get_jit_include_dir, get_offload_arch
    from yan_amd.jit_kernels import bf16_gemm
    dtype = getattr(torch, dtype_name)
    _, keys, arg_defs = bf16_gemm.dense_kernel_plan(*shape, dtype, 256, 0)
    assert keys['BLOCK_M'] == 256 and keys['NUM_STAGES'] == 2             # the 8-wave kernel
    src, asm = tmp_path / 'kernel.cu', tmp_path / 'kernel.s'
    src.write_text(generate(bf16_gemm.includes, arg_defs, cpp_format(bf16_gemm.template, keys)))
    subprocess.check_call([get_hipcc_compiler()[0], '-x', 'hip', '--cuda-device-only', '-S', '-std=c++20', '-O3',
                           f'--offload-arch={get_offload_arch()}', '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
                           f'-I{get_jit_include_dir()}', str(src), '-o', str(asm)])
    text = asm.read_text()
    assert re.search(r'\.private_segment_fixed_size:\s+0\b', text), 'the kernel spills'
    # instructions and labels of the kernel, in text order
    lines = [line.split(';')[0].strip() for line in text.split('\n')]
    lines = [line for line in lines if line and (line.endswith(':') or not line.startswith(('.', '//')))]

    def regs(operand_text):
        found = set()
        for lo, hi in re.findall(r'\bv\[(\d+):(\d+)\]', operand_text):
            found.update(range(int(lo), int(hi) + 1))
        found.update(int(r) for r in re.findall(r'\bv(\d+)\b', operand_text))
        return found

    mfma = re.compile(r'^v_mfma_f32_16x16x32_(?:bf16|f16) (v\[\d+:\d+\]), (v\[\d+:\d+\]), (v\[\d+:\d+\]), (v\[\d+:\d+\])')
    where = [i for i, line in enumerate(lines) if mfma.match(line)]
    assert len(where) >= 2 * 2 * keys['BLOCK_N'] // 32 * 4          # at least the steps of two k-tiles
    acc = set()
    for i in where:
        dst, a, b, c = mfma.match(lines[i]).groups()
        assert dst == c, lines[i]                                    # accumulates in place
        acc |= regs(dst)
    assert len(acc) == 256 * keys['BLOCK_N'] // 512                  # one register per output of the wave's slab
    for i in where:
        _, a, b, _ = mfma.match(lines[i]).groups()
        assert not (regs(a) | regs(b)) & acc, lines[i]

    def mfma_in_flight_before(i):
        """An MFMA less than 20 instructions up the straight-line path that ends at instruction i, with no `s_nop 15`
        pair between; a path stops at a label whose predecessor in the text ends with an unconditional branch."""
        nops = 0
        for back in range(1, 21):
            line = lines[i - back]
            if line.endswith(':'):
                if lines[i - back - 1].startswith('s_branch'):
                    return False
                continue
            if line == 's_nop 15':
                nops += 1
            if mfma.match(line):
                return nops < 2
        return False
    for i in range(where[0], len(lines)):
        line = lines[i]
        if mfma.match(line) or line.endswith(':') or line.startswith('s_') or not regs(line) & acc:
            continue
        assert not mfma_in_flight_before(i), f'{line} touches an accumulator right behind an MFMA'
    # and the epilogue's first read of a sum sits behind the wait states written in the source
    after = lines[where[-1] + 1:]
    first_use = next(i for i, line in enumerate(after) if not line.endswith(':') and not line.startswith('s_') and regs(line) & acc)
    assert sum(1 for line in after[:first_use] if line == 's_nop 15') >= 2, 'the sums are read before the last MFMAs have retired'


@pytest.mark.parametrize('dtype_name', ['bfloat16', 'half'])
def test_the_4_wave_dense_kernel_keeps_its_sums_in_place_and_one_instruction_behind_each_mfma(tmp_path, dtype_name):
    """The 4-wave kernel of the 256 x 256 tile has one wave per SIMD: a spill, a sum that wanders, or two memory instructions
    back to back in its main loop leave the matrix core idle. Checked on the generated code (compiled for the device only):
    no scratch; every MFMA adds into the accumulation registers it reads (or starts them from zero), 256 of them; in the
    main loop an MFMA sits between any two copies or fragment reads; the epilogue reads
    the sums behind the wait states written in the source."""
    import re
    import subprocess
    from yan_amd.jit import cpp_format, generate
    from yan_amd.jit.compiler import get_hipcc_compiler, get_jit_include_dir, get_offload_arch
    from yan_amd.jit_kernels import bf16_gemm
    dtype = getattr(torch, dtype_name)
    _, keys, arg_defs = bf16_gemm.dense_kernel_plan(8192, 8192, 8192, dtype, 256, 0)
    assert (keys['BLOCK_M'], keys['BLOCK_N'], keys['NUM_STAGES']) == (256, 256, 2)
    src, asm = tmp_path / 'kernel.cu', tmp_path / 'kernel.s'
    src.write_text(generate(bf16_gemm.includes, arg_defs, cpp_format(bf16_gemm.template, keys)))
    subprocess.check_call([get_hipcc_compiler()[0], '-x', 'hip', '--cuda-device-only', '-S', '-std=c++20', '-O3',
                           f'--offload-arch={get_offload_arch()}', '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
                           f'-I{get_jit_include_dir()}', str(src), '-o', str(asm)])
    text = asm.read_text()
    assert set(re.findall(r'\.private_segment_fixed_size:\s+(\d+)', text)) == {'0'} and 'scratch_' not in text, 'a kernel spills'
    name = 'dense_gemm_mfma_4w' if dtype == torch.bfloat16 else 'fp16_gemm_cute_4w'
    start = next(i for i, line in enumerate(text.split('\n')) if re.match(rf'^_ZN3yan\d*{name}\w*:', line))
    lines = [line.split(';')[0].strip() for line in text.split('\n')[start + 1:]]
    lines = lines[:lines.index('s_endpgm')]
    lines = [line for line in lines if line and not line.startswith(('.', '//'))]
    mfma = re.compile(r'^v_mfma_f32_16x16x32_(?:bf16|f16) (a\[\d+:\d+\]), v\[\d+:\d+\], v\[\d+:\d+\], (a\[\d+:\d+\]|0)$')
    assert not [line for line in lines if line.startswith('v_mfma') and not mfma.match(line)]
    sums = set()
    for line in lines:
        found = mfma.match(line)
        if found:
            assert found.group(2) in (found.group(1), '0'), line
            lo, hi = map(int, re.match(r'a\[(\d+):(\d+)\]', found.group(1)).groups())
            sums.update(range(lo, hi + 1))
    assert sums == set(range(256))
    # the main loop: from the second barrier (the first opens the first k-tile of the walk) to the last MFMA
    barriers = [i for i, line in enumerate(lines) if line == 's_barrier']
    last_mfma = max(i for i, line in enumerate(lines) if mfma.match(line))
    loop = [line for line in lines[barriers[1] + 1:last_mfma + 1] if not line.startswith('s_') and not line.endswith(':')]
    heavy = [i for i, line in enumerate(loop) if line.startswith(('buffer_load', 'ds_read'))]
    assert len(heavy) >= (16 + 32) + (8 + 16)              # a k-tile of the loop and the second k-half of the first one
    assert all(any(mfma.match(line) for line in loop[i + 1:j]) for i, j in zip(heavy, heavy[1:])), 'two copies or fragment reads with no MFMA between them'
    after = lines[last_mfma + 1:]
    first_read = next(i for i, line in enumerate(after) if line.startswith('v_accvgpr_read'))
    assert sum(1 for line in after[:first_read] if line == 's_nop 15') >= 2


@pytest.mark.parametrize('shape', [(4096, 7168, 7168), (64, 4096, 7168), (4096, 5120, 5120)])
def test_fp8_kernels_of_the_baseline_shapes_do_not_spill(tmp_path, shape):
    """The FP8 main loop keeps 128 running sums, the fragments of a row of atoms and the scales in registers and sits close
    to the 256-register limit; a spill puts scratch loads among its copies, and every wait for one of them waits for all
    copies in flight (measured: a variant that spilled 260 bytes ran 2.3 times slower). Checked on the generated code,
    compiled for the device only."""
    import re
    import subprocess
    from yan_amd.jit import cpp_format, generate
    from yan_amd.jit.compiler import get_hipcc_compiler, get_jit_include_dir, get_offload_arch
    _, keys, arg_defs, _, code_template = gemm.fp8_kernel_plan(*shape, 256, True)
    src, asm = tmp_path / 'kernel.cu', tmp_path / 'kernel.s'
    src.write_text(generate(gemm.includes, arg_defs, cpp_format(code_template, keys)))
    subprocess.check_call([get_hipcc_compiler()[0], '-x', 'hip', '--cuda-device-only', '-S', '-std=c++20', '-O3',
                           f'--offload-arch={get_offload_arch()}', '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
                           f'-I{get_jit_include_dir()}', str(src), '-o', str(asm)])
    text = asm.read_text()
    assert re.findall(r'\.private_segment_fixed_size:\s+(\d+)', text) == ['0'], 'the kernel spills'
    assert 'scratch_' not in text
    assert all(int(n) <= 256 for n in re.findall(r'\.vgpr_count:\s+(\d+)', text))
    assert text.count('16x16x128_f8f6f4') >= 4


def test_tuner_rebuilds_when_a_callers_dict_changes_between_calls(monkeypatch):
    """A caller that reuses one mutable keys dict (the loop of the reference's tests/test_jit.py) gets the kernel of the
    keys it passes, not of the keys it passed last time; only read-only plan keys take the same-object short cut."""
    from yan_amd.jit_kernels import tuner as tuner_mod
    built = []

    def fake_build(name, arg_defs, code):
        built.append(code)
        return object()
    monkeypatch.setattr(tuner_mod, 'build', fake_build)
    t = tuner_mod.JITTuner()
    kw = dict(name='k', space=(), includes=(), arg_defs=(('x', int),), template='int v = {V};', args=(1,))
    keys = {'V': 1}
    first = t.compile_and_tune(keys=keys, **kw)
    assert t.compile_and_tune(keys=keys, **kw) is first and len(built) == 1
    keys['V'] = 2
    second = t.compile_and_tune(keys=keys, **kw)
    assert second is not first and len(built) == 2 and 'int v = 2;' in built[1]
    frozen = tuner_mod.FrozenKeys({'V': 1})
    assert t.compile_and_tune(keys=frozen, **kw) is first and t.compile_and_tune(keys=frozen, **kw) is first
    with pytest.raises(TypeError):
        frozen['V'] = 3


def test_compare_tensors_verdicts(capsys):
    """yan/jit_kernels/utils.py:138-179: element-wise and similarity modes, shape mismatch, unknown mode."""
    from yan_amd.jit_kernels import compare_tensors
    x = torch.arange(12, dtype=torch.float32).view(3, 4)
    assert compare_tensors(x, x.clone()) is True and compare_tensors(x, x.clone(), mode='similarity', verbose=False) is True
    y = x.clone()
    y[1, 2] += 0.5
    capsys.readouterr()
    assert compare_tensors(y, x, verbose=False) is False
    said = capsys.readouterr().out
    assert 'FAILED' in said and 'Max diff: 0.500000' in said and '[1, 2]' in said and 'Actual tensor' not in said
    assert compare_tensors(y, x, atol=1.0) is True
    assert compare_tensors(y, x, mode='similarity', diff_tolerance=1e-2) is True
    assert compare_tensors(y, x, mode='similarity', diff_tolerance=1e-9) is False
    assert compare_tensors(torch.zeros(3), torch.zeros(3), mode='similarity') is True
    assert compare_tensors(x, x[:2]) is False and compare_tensors(x, x, mode='cosine') is False


def test_split_k_workspaces_are_kept_per_stream_and_per_capture():
    """Bookkeeping of the Python entries' split-K workspaces: eager launches share a workspace per (device, stream), at
    most `max_eager` are kept; every capture gets its own, never shared with eager launches or another capture and never
    dropped; a workspace whose launch failed is cleared before its next use."""
    from yan_amd.jit_kernels.split_k import WorkspaceBook
    made, cleared = [], []
    book = WorkspaceBook(make=lambda: made.append(object()) or made[-1], clear=cleared.append, max_eager=3)
    w0 = book.get(0, 111)
    assert book.get(0, 111) is w0 and len(made) == 1
    w1 = book.get(0, 222)
    w2 = book.get(1, 111)
    assert len({id(w) for w in (w0, w1, w2)}) == 3
    # captures: keyed by the capture's id, not by the stream that records it
    c7 = book.get(0, 111, capture=7)
    assert c7 is not w0 and book.get(0, 111, capture=7) is c7 and book.get(0, 999, capture=7) is c7
    c8 = book.get(0, 111, capture=8)
    assert c8 is not c7 and book.get(1, 111, capture=7) is not c7
    assert len(made) == 6 and not cleared
    # a failed launch: cleared once, at the next use
    book.launch_failed(0, 222)
    assert not cleared
    assert book.get(0, 222) is w1 and cleared == [w1]
    assert book.get(0, 222) is w1 and cleared == [w1]
    book.launch_failed(0, 111, capture=7)           # the graph's own first node zeroes a capture's workspace
    assert book.get(0, 111, capture=7) is c7 and cleared == [w1]
    # eviction: the oldest eager workspace goes, captures stay
    book.launch_failed(0, 111)
    w3 = book.get(2, 5)
    assert (0, 111) not in book.eager and len(book.eager) == 3 and (0, 111) not in book.suspect
    assert book.get(0, 111) is not w0 and cleared == [w1]       # a fresh one: nothing to clear
    assert len(book.captures) == 3 and book.get(0, 1, capture=8) is c8 and w3 is book.get(2, 5)


def test_the_bf16_activation_entry_chains_the_quantiser_in_front_of_whatever_the_gemm_entry_runs():
    """`fp8_cast_chain_plan`: the keys of the GEMM plan the FP8 entry uses for the sizes (split-K plan, weight-streaming kernel
    or tiles) plus the scratch offset, a `launch` whose arguments are the GEMM's without the quantised operands, and code
    that calls the quantiser before the GEMM's launch; None when the codes do not fit the scratch."""
    import harness as testing
    from yan_amd.jit import cpp_format
    from yan_amd.jit_kernels.split_k import SPLIT_K_WORKSPACE_BYTES, WORKSPACE_ALLOCATION_BYTES
    assert WORKSPACE_ALLOCATION_BYTES == SPLIT_K_WORKSPACE_BYTES + gemm.CAST_SCRATCH_BYTES
    for m, n, k in testing.CAST_CHAIN_SHAPES:
        plan = gemm.fp8_cast_chain_plan(m, n, k, 256)
        if m * k + m * (k // 128) * 4 + 256 > gemm.CAST_SCRATCH_BYTES:
            assert plan is None
            continue
        name, keys, arg_defs, code_template, smem_size = plan
        split = gemm.fp8_split_k_plan(m, n, k, 256, True)
        inner_keys, inner_defs = (split[1], split[2]) if split is not None else gemm.fp8_kernel_plan(m, n, k, 256, True)[1:3]
        assert name == 'gemm_bf16_fp8_bf16_nt' and dict(keys) == {**inner_keys, 'SCRATCH_OFFSET': SPLIT_K_WORKSPACE_BYTES}
        assert [d[0] for d in arg_defs] == ['x', 'buffer', 'scratch_bytes'] + [d[0] for d in inner_defs if d[0] not in ('lhs', 'lhs_scales')]
        code = cpp_format(code_template, keys)
        assert code.index('launch_per_token_cast(') < code.index('__return_code = static_cast<int>(', code.index('launch_per_token_cast(') + 1)
        assert '{' + 'SCRATCH_OFFSET' + '}' not in code and smem_size > 0
    # without split-K (YAN_SPLIT_K=0 leaves the entries without memory of their own) the entry makes two calls; the plan for it is not asked
    assert gemm.fp8_cast_chain_plan(64, 4096, 7168, 256, False)[1].get('SPLIT_K') is None
