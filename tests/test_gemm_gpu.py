"""Parity of the HIP GEMMs against the CPU oracle, through the JIT boundary (`launch` in a cached kernel.so).

bf16 / fp16: calc_diff < 1e-5 against the fp32 matmul of the same 16-bit inputs.
FP8:         calc_diff < 1e-3 against the fp32 matmul of the dequantised operands; exactly representable cases
             must match bit for bit.
Sizes the oracle finishes in seconds are compared in full; the baseline sizes are checked on a seeded sample of
rows against the oracle, in full against a chunked fp32 matmul on the device, and through size-independent
properties (exact linearity in power-of-two scales, layout independence of the scale tensor).
"""
import os
import sys

import numpy as np
import pytest
import torch

import oracle
import yan_amd as yan
import harness as testing
from yan_amd import capi, jit

pytestmark = pytest.mark.gpu

BF16_TOL, FP8_TOL = 1e-5, 1e-3


def _announce(*what):
    print('[case]', *what, flush=True)
    sys.stdout.flush()


def _np(t):
    if t.dtype == torch.float8_e4m3fn:
        return t.view(torch.uint8).cpu().numpy()
    return t.float().cpu().numpy()


@pytest.fixture(scope='module', autouse=True)
def _device():
    assert torch.cuda.is_available(), 'these tests need a GPU'
    torch.cuda.set_device(0)
    yield
    torch.cuda.synchronize()


# ----------------------------------------------------------------------------- the boundary itself
def test_jit_boundary_known_answer(capfd):
    """tests/test_jit.py:31-64 of the reference: the six arguments arrive in `launch` as passed."""
    args = (('lhs', torch.float8_e4m3fn), ('rhs', torch.float8_e4m3fn), ('scale', torch.float), ('out', torch.bfloat16),
            ('enable_double_streams', bool), ('stream', torch.cuda.Stream))
    body = '\n' + ''.join(f'std::cout << reinterpret_cast<uint64_t>({n}) << std::endl;\n' for n in ('lhs', 'rhs', 'scale', 'out'))
    body += 'std::cout << enable_double_streams << std::endl;\nstd::cout << reinterpret_cast<uint64_t>(stream) << std::endl;\n'
    func = jit.build('test_func', args, jit.generate((), args, body))
    fp8 = torch.empty((1,), dtype=torch.float8_e4m3fn, device='cuda')
    fp32 = torch.empty((1,), dtype=torch.float, device='cuda')
    bf16 = torch.empty((1,), dtype=torch.bfloat16, device='cuda')
    stream = torch.cuda.current_stream()
    capfd.readouterr()
    assert func(fp8, fp8, fp32, bf16, True, stream) == 0
    out = capfd.readouterr().out
    assert out == f'{fp8.data_ptr()}\n{fp8.data_ptr()}\n{fp32.data_ptr()}\n{bf16.data_ptr()}\n1\n{stream.cuda_stream}\n'


def test_launch_reports_bad_sizes_through_the_return_code():
    from yan_amd.jit_kernels import bf16_gemm
    name, keys, defs = bf16_gemm.dense_kernel_plan(64, 64, 64, torch.bfloat16, 256)
    rt = jit.build(name, defs, jit.generate(bf16_gemm.includes, defs, jit.cpp_format(bf16_gemm.template, keys)))
    a = torch.zeros(64, 64, dtype=torch.bfloat16, device='cuda')
    assert rt(64, 64, 64, a, a, a, torch.cuda.current_stream()) == 0
    assert rt(64, 62, 64, a, a, a, torch.cuda.current_stream()) != 0        # n % 4 != 0
    assert rt(64, 64, 60, a, a, a, torch.cuda.current_stream()) != 0        # k % 8 != 0
    assert rt(-1, 64, 64, a, a, a, torch.cuda.current_stream()) != 0
    torch.cuda.synchronize()


# ----------------------------------------------------------------------------- bf16 / fp16
@pytest.mark.parametrize('m,n,k', [s for s in testing.DENSE_TEST_SHAPES if s[0] * s[1] * s[2] <= 7e10])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.half])
def test_dense_parity_vs_oracle(m, n, k, dtype):
    _announce('dense', dtype, m, n, k)
    a, b, c = testing.make_bf16_case(m, n, k, seed=42, dtype=dtype, device='cuda')
    c.fill_(float('nan'))
    (yan.gemm_bf16_tn if dtype == torch.bfloat16 else yan.gemm_fp16_tn)(a, b, c)
    torch.cuda.synchronize()
    got = _np(c)
    assert np.isfinite(got).all()
    ref = oracle.gemm_bf16_tn_ref(_np(a), _np(b))
    assert oracle.calc_diff(got, ref) < BF16_TOL
    # every element within one output rounding step of the fp32 result (plus fp32 accumulation slack)
    ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
    assert bool(np.all(np.abs(got - ref) <= np.abs(ref) * ulp + 1e-4 * np.sqrt(k)))


def test_dense_golden_fixture(repo_root):
    z = np.load(os.path.join(repo_root, 'tests', 'golden', 'gemm_small.npz'))
    a = torch.from_numpy(z['bf16_a_bits'].view(np.int16)).view(torch.bfloat16).cuda()
    b = torch.from_numpy(z['bf16_b_bits'].view(np.int16)).view(torch.bfloat16).cuda()
    c = torch.zeros(a.size(0), b.size(0), dtype=torch.bfloat16, device='cuda')
    yan.gemm_bf16_tn(a, b, c)
    assert oracle.calc_diff(_np(c), z['bf16_expected_f64']) < BF16_TOL
    # the kernel's fp32 sum, rounded once to bf16, is within one bf16 step of the correctly rounded fp64 value
    want = oracle.bf16_round(z['bf16_expected_f64'].astype(np.float32))
    assert np.all(np.abs(_np(c) - want) <= np.abs(want) * 2.0 ** -7 + 1e-6)


def test_dense_closed_forms_are_exact():
    # ones pattern of the reference's smoke case (yan/jit_kernels/cute_gemm.py:74-79): c == ceil(k / 12) everywhere
    m, n, k = 128, 256, 256
    a = torch.zeros(m, k, dtype=torch.bfloat16, device='cuda')
    b = torch.zeros(n, k, dtype=torch.bfloat16, device='cuda')
    a[:, ::4] = 1.0
    b[:, ::3] = 1.0
    c = torch.zeros(m, n, dtype=torch.bfloat16, device='cuda')
    yan.gemm_bf16_tn(a, b, c)
    assert torch.equal(c, torch.full_like(c, -(-k // 12)))
    # identity weights return the activations bit for bit; catches transposed or permuted operands
    g = torch.Generator().manual_seed(3)
    a = torch.randn(300, 256, generator=g).bfloat16().cuda()
    eye = torch.eye(256, dtype=torch.bfloat16, device='cuda')
    c = torch.zeros(300, 256, dtype=torch.bfloat16, device='cuda')
    yan.gemm_bf16_tn(a, eye, c)
    assert torch.equal(c, a)
    # untouched memory around a ragged output stays untouched
    big = torch.full((70, 136), 7.0, dtype=torch.bfloat16, device='cuda')
    a, b, _ = testing.make_bf16_case(33, 132, 72, seed=5, device='cuda')
    out = big[:33 * 132 // 136 + 1].view(-1)[:33 * 132].view(33, 132)
    yan.gemm_bf16_tn(a, b, out)
    assert torch.all(big.view(-1)[33 * 132:] == 7.0)
    assert oracle.calc_diff(_np(out), oracle.gemm_bf16_tn_ref(_np(a), _np(b))) < BF16_TOL


@pytest.mark.parametrize('m,n,k', [(7, 1156, 512), (20, 100, 2112)])
def test_dense_weight_streaming_kernel_leaves_its_neighbours_alone(m, n, k):
    """A handful of rows runs one workgroup per 16 weight rows, the last one partly past n: rows from m on and the columns
    past n of the last workgroup stay untouched, JIT entry and C library give the same bits."""
    from yan_amd.jit_kernels import heuristics
    _announce('dense weight streaming', m, n, k)
    assert heuristics.get_dense_tile(m, n, k, yan.get_num_sms())[1] == 16
    a, b, _ = testing.make_bf16_case(m, n, k, seed=6, device='cuda')
    big = torch.full((m + 2, n), 7.0, dtype=torch.bfloat16, device='cuda')
    # built from its plan: where K is long enough the public entry point prefers a split-K plan to the two-atom kernel
    from yan_amd.jit_kernels import bf16_gemm
    name, keys, defs = bf16_gemm.dense_kernel_plan(m, n, k, torch.bfloat16, yan.get_num_sms())
    assert keys['BLOCK_N'] == 16
    runtime = jit.build(name, defs, jit.generate(bf16_gemm.includes, defs, jit.cpp_format(bf16_gemm.template, keys)))
    assert runtime(m, n, k, a, b, big[:m], torch.cuda.current_stream()) == 0
    torch.cuda.synchronize()
    assert bool((big[m:] == 7.0).all())
    assert oracle.calc_diff(_np(big[:m]), oracle.gemm_bf16_tn_ref(_np(a), _np(b))) < BF16_TOL
    again = torch.empty(m, n, dtype=torch.bfloat16, device='cuda')
    assert capi.gemm_bf16_tn(a, b, again) == 0
    assert torch.equal(again, big[:m])


@pytest.mark.parametrize('m,n,k', testing.DENSE_SPLIT_K_SHAPES)
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.half])
def test_dense_split_k_parity_vs_oracle(m, n, k, dtype):
    """Problems whose K the dense entry points split over 2 to 4 workgroups per tile (the three tiles, every factor, ragged
    edges, a k tail): parity against the oracle to the bar of the unsplit kernels, the same bits from the library's split-K
    entry point, which writes nothing past row m, and arrival counters back at zero."""
    from yan_amd.jit_kernels import bf16_gemm
    plan = bf16_gemm.dense_split_k_plan(m, n, k, dtype, yan.get_num_sms())
    assert plan is not None and (plan[1]['BLOCK_M'], plan[1]['BLOCK_N'], plan[1]['SPLIT_K']) == testing.DENSE_SPLIT_K_PLAN_OF_SHAPE[(m, n, k)]
    _announce('dense split-k', dtype, m, n, k, plan[1]['BLOCK_M'], plan[1]['BLOCK_N'], plan[1]['SPLIT_K'])
    a, b, c = testing.make_bf16_case(m, n, k, seed=42, device='cuda', dtype=dtype)
    c.fill_(float('nan'))
    (yan.gemm_bf16_tn if dtype == torch.bfloat16 else yan.gemm_fp16_tn)(a, b, c)
    torch.cuda.synchronize()
    got, ref = _np(c), oracle.gemm_bf16_tn_ref(_np(a), _np(b))
    assert np.isfinite(got).all()
    assert oracle.calc_diff(got, ref) < BF16_TOL
    ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
    assert bool(np.all(np.abs(got - ref) <= np.abs(ref) * ulp + 1e-4 * np.sqrt(k)))
    workspace = capi.split_k_workspace()
    padded = torch.full((m + 3, n), 7.0, dtype=dtype, device='cuda')
    assert capi.gemm_bf16_tn_split_k(a, b, padded, workspace) == 0
    torch.cuda.synchronize()
    assert torch.equal(padded[:m], c) and bool((padded[m:] == 7.0).all())
    counters = capi.load().yan_gemm_split_k_counter_bytes()
    assert int(workspace[:counters].view(torch.int32).abs().sum()) == 0


def test_dense_baseline_8192_cubed():
    """cfg2: rows sampled against the oracle, the whole matrix against a chunked fp32 matmul on the device."""
    m = n = k = 8192
    _announce('dense cfg2', m, n, k)
    a, b, c = testing.make_bf16_case(m, n, k, seed=42, scale=k ** -0.5, device='cuda', gen_device='cuda')
    yan.gemm_bf16_tn(a, b, c)
    rows = np.random.default_rng(0).choice(m, 64, replace=False)
    ref = oracle.gemm_bf16_tn_ref(_np(a[rows]), _np(b))
    assert oracle.calc_diff(_np(c[rows]), ref) < BF16_TOL
    num = den = 0.0
    for r0 in range(0, m, 1024):
        ref = a[r0:r0 + 1024].float() @ b.float().t()
        got = c[r0:r0 + 1024].float()
        num += (got.double() * ref.double()).sum().item()
        den += (got.double() ** 2 + ref.double() ** 2).sum().item()
    assert 1 - 2 * num / den < BF16_TOL


@pytest.mark.parametrize('m,n,k', [(8192, 4096, 14336), (12100, 12200, 12288)])
def test_dense_beyond_the_memory_side_cache_walks_regions(m, n, k):
    """Operands of more than 256 MB put the 256 x 256 kernel's tile walk into region order (16 x 16 tiles per round for the
    first shape, 32 x 8 with ragged edges for the second): every 512-row block of the output against a chunked fp32
    matmul on the device, so that a tile written to the wrong place, twice or not at all fails its block."""
    _announce('dense beyond the cache', m, n, k)
    from yan_amd.jit_kernels import bf16_gemm
    assert bf16_gemm.dense_kernel_plan(m, n, k, torch.bfloat16, yan.get_num_sms(), 0)[1]['BLOCK_M'] == 256
    a, b, c = testing.make_bf16_case(m, n, k, seed=9, scale=k ** -0.5, device='cuda', gen_device='cuda')
    c.fill_(float('nan'))
    yan.gemm_bf16_tn(a, b, c)
    bt = b.float().t()
    for r0 in range(0, m, 512):
        ref = (a[r0:r0 + 512].float() @ bt).double()
        got = c[r0:r0 + 512].double()
        diff = 1 - 2 * (got * ref).sum().item() / ((got * got).sum().item() + (ref * ref).sum().item())
        assert diff < BF16_TOL, (r0, diff)


def _explicit_dense_runtime(tile, dtype=torch.bfloat16, eight_waves=False):
    from yan_amd.jit_kernels import bf16_gemm
    name, keys, defs, template = testing.dense_explicit_plan(tile, dtype, eight_waves)
    return jit.build(name, defs, jit.generate(bf16_gemm.includes, defs, jit.cpp_format(template, keys)))


@pytest.mark.parametrize('m,n,k', testing.DENSE_SEEDED_BOTH_KERNELS_SHAPES)
def test_both_kernels_agree_on_every_tile_width_for_seeded_shapes(m, n, k):
    """Every 256-row tile width in turn with the tile given, so that shapes the cost model would never hand to a width reach it
    too (a single row, eight columns, far fewer tiles than compute units): the 4-wave and the 8-wave kernel give the same
    bits, nothing outside the matrix is touched, and the result agrees with the oracle."""
    _announce('dense, both kernels, tile given', torch.bfloat16, m, n, k)
    a, b, c = testing.make_bf16_case(m, n, k, seed=m + n + k, device='cuda')
    ref = oracle.gemm_bf16_tn_ref(_np(a), _np(b))
    for block_n in (160, 192, 224, 256):
        four, eight = _explicit_dense_runtime((256, block_n)), _explicit_dense_runtime((256, block_n), eight_waves=True)
        # one allocation with a guard row behind the matrix: the kernels address rows past m through their descriptors
        whole = torch.full((m + 1, n), float('nan'), dtype=torch.bfloat16, device='cuda')
        got, want = whole[:m], torch.full_like(c, float('nan'))
        assert four(m, n, k, a, b, got, torch.cuda.current_stream()) == 0
        assert eight(m, n, k, a, b, want, torch.cuda.current_stream()) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want), block_n
        assert bool(torch.isnan(whole[m]).all()), block_n
        assert oracle.calc_diff(_np(got), ref) < BF16_TOL, block_n


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.half])
@pytest.mark.parametrize('m,n,k', testing.DENSE_BOTH_KERNELS_SHAPES)
def test_both_kernels_of_the_256_row_tiles_give_the_same_bits(m, n, k, dtype):
    """The launcher of the tiles of 256 rows and 160 to 256 columns takes the 4-wave kernel when K is whole k-tiles, at least
    four of them, and n a multiple of 8, the 8-wave kernel otherwise: same walk over the tiles, same K rotation, same order
    of summation, so the same bits, also under a cap on the workgroups; and against the oracle."""
    _announce('dense, both kernels', dtype, m, n, k)
    from yan_amd.jit_kernels import bf16_gemm
    name, keys, defs = bf16_gemm.dense_kernel_plan(m, n, k, dtype, yan.get_num_sms(), 0)
    assert keys['BLOCK_M'] == 256 and keys['BLOCK_N'] >= 160
    a, b, c = testing.make_bf16_case(m, n, k, seed=11, dtype=dtype, device='cuda')
    c.fill_(float('nan'))
    entry = yan.gemm_bf16_tn if dtype == torch.bfloat16 else yan.gemm_fp16_tn
    entry(a, b, c)
    eight = _explicit_dense_runtime((keys['BLOCK_M'], keys['BLOCK_N']), dtype, eight_waves=True)
    want = torch.full_like(c, float('nan'))
    assert eight(m, n, k, a, b, want, torch.cuda.current_stream()) == 0
    torch.cuda.synchronize()
    assert torch.equal(c, want)
    ref = oracle.gemm_bf16_tn_ref(_np(a), _np(b))
    assert oracle.calc_diff(_np(c), ref) < BF16_TOL
    # the same tile on fewer workgroups than compute units (a cap set through the entry would also change the tile choice)
    for cap in (7, 100):
        name, capped_keys, defs = bf16_gemm.dense_kernel_plan(m, n, k, dtype, yan.get_num_sms(), cap)
        assert capped_keys['NUM_SMS'] == cap and capped_keys['BLOCK_N'] == keys['BLOCK_N']
        capped = jit.build(name, defs, jit.generate(bf16_gemm.includes, defs, jit.cpp_format(bf16_gemm.template, capped_keys)))
        again = torch.full_like(c, float('nan'))
        assert capped(m, n, k, a, b, again, torch.cuda.current_stream()) == 0
        torch.cuda.synchronize()
        assert torch.equal(again, c), cap
    # which kernel ran: by its name in the profiler
    kernel = 'dense_gemm_mfma_4w' if dtype == torch.bfloat16 else 'fp16_gemm_cute_4w'
    assert yan.bench_kineto(lambda: entry(a, b, c), kernel, num_tests=2, suppress_kineto_output=True) > 0


# ----------------------------------------------------------------------------- FP8 block-scaled
def _fp8_ref(a8, sa, b8, sb):
    return oracle.gemm_fp8_block_scaled_ref(_np(a8), sa.cpu().numpy(), _np(b8), sb.cpu().numpy())


@pytest.mark.parametrize('m,n,k', testing.REFERENCE_DENSE_TEST_SHAPES)
def test_fp16_entry_on_the_reference_test_shapes(m, n, k):
    """The flow of the reference's dense test (tests/test_cute.py:9-27): fp16 randn operands, zeroed output,
    `gemm_fp16_tn`, calc_diff < 1e-3 against torch's own fp16 `x @ y.t()`; and the bar of this build, < 1e-5 against
    the fp32 product of the same operands."""
    g = torch.Generator(device='cuda').manual_seed(42 + m + n + k)
    x = torch.randn(m, k, device='cuda', dtype=torch.half, generator=g)
    y = torch.randn(n, k, device='cuda', dtype=torch.half, generator=g)
    out = torch.zeros(m, n, device='cuda', dtype=torch.half)
    assert yan.gemm_fp16_tn(x, y, out) is None
    assert float(yan.calc_diff(out, x @ y.t())) < 1e-3
    assert float(yan.calc_diff(out.float(), x.float() @ y.float().t())) < 1e-5


def test_fp16_kernel_answers_to_the_reference_kernel_name():
    """tests/test_cute.py:35 times the kernel whose name contains 'fp16_gemm_cute'; the reference's package-level
    smoke check is reachable under its name as well (yan/jit_kernels/__init__.py:2)."""
    m, n, k = 256, 5120, 5120
    x = torch.randn(m, k, device='cuda', dtype=torch.half)
    y = torch.randn(n, k, device='cuda', dtype=torch.half)
    out = torch.zeros(m, n, device='cuda', dtype=torch.half)
    t = yan.bench_kineto(lambda: yan.gemm_fp16_tn(x, y, out), 'fp16_gemm_cute', suppress_kineto_output=True)
    assert 0 < t < 1e-3
    assert yan.jit_kernels.cute_gemm_accuracy_test is yan.jit_kernels.bf16_gemm_accuracy_test


# ----------------------------------------------------------------------------- fp32 GEMM with alpha / beta
FLOAT_TOL = 1e-10       # calc_diff against the fp64 product; fp32 accumulation of N(0,1) data sits near 1e-14


def _float_close(got, want, k):
    return np.allclose(got, want, rtol=1e-5, atol=1e-5 * max(1.0, float(np.abs(want).max())))


@pytest.mark.parametrize('m,n,k', testing.FLOAT_TEST_SHAPES)
def test_float_gemm_parity_vs_oracle_with_alpha_beta(m, n, k):
    _announce('fp32', m, n, k)
    a, b, c = testing.make_float_case(m, n, k, seed=5, device='cuda')
    assert yan.gemm_float_nt(a, b, c) is None
    want = oracle.gemm_float_nt_ref(_np(a), _np(b))
    assert oracle.calc_diff(_np(c), want) < FLOAT_TOL and _float_close(_np(c), want, k)
    # alpha and beta: c <- alpha * a b^T + beta * c, on top of what the first call left
    before = _np(c)
    yan.gemm_float_nt(a, b, c, alpha=-0.5, beta=2.0)
    want2 = oracle.gemm_float_nt_ref(_np(a), _np(b), before, -0.5, 2.0)
    assert oracle.calc_diff(_np(c), want2) < FLOAT_TOL and _float_close(_np(c), want2, k)
    # beta == 0 does not read c: NaNs in it do not propagate
    c.fill_(float('nan'))
    yan.gemm_float_nt(a, b, c, alpha=1.0, beta=0.0)
    assert oracle.calc_diff(_np(c), want) < FLOAT_TOL


@pytest.mark.parametrize('m,n,k', testing.REFERENCE_FLOAT_TEST_SHAPES)
def test_float_entry_on_the_reference_test_shapes(m, n, k):
    """The flow of the reference's fp32 test (tests/test_simple.py:9-27): randn operands made col-major with
    `get_col_major_tensor`, zeroed output, `gemm_float_nt`, calc_diff < 1e-3 against `x @ y.t()`; and the bar of this
    build: 1e-10 against the fp64 product on the device and against the oracle on a seeded sample of rows."""
    _announce('fp32 reference shape', m, n, k)
    g = torch.Generator(device='cuda').manual_seed(42 + m + n + k)
    x = torch.randn(m, k, device='cuda', dtype=torch.float32, generator=g)
    y = torch.randn(n, k, device='cuda', dtype=torch.float32, generator=g)
    out = torch.zeros(m, n, device='cuda', dtype=torch.float32)
    ref_out = x @ y.t()
    assert yan.gemm_float_nt(yan.get_col_major_tensor(x), yan.get_col_major_tensor(y), out) is None
    assert float(yan.calc_diff(out, ref_out)) < 1e-3
    assert float(yan.calc_diff(out.double(), x.double() @ y.double().t())) < FLOAT_TOL
    rows = np.random.default_rng(m + n + k).choice(m, size=8, replace=False)
    want = oracle.gemm_float_nt_ref(_np(x[rows]), _np(y))
    assert oracle.calc_diff(_np(out[rows]), want) < FLOAT_TOL and _float_close(_np(out[rows]), want, k)


def test_float_gemm_closed_forms_are_exact_and_kernel_name():
    # the ones pattern: c = ceil(k / 12) everywhere, exactly; alpha = 0.5, beta = -2 on top of it stays exact
    m, n, k = 256, 320, 252
    a, b = torch.zeros(k, m, device='cuda').t(), torch.zeros(k, n, device='cuda').t()
    a[:, ::4] = 1
    b[:, ::3] = 1
    c = torch.zeros(m, n, device='cuda')
    yan.gemm_float_nt(a, b, c)
    assert torch.equal(c, torch.full_like(c, 21.0))
    yan.gemm_float_nt(a, b, c, alpha=0.5, beta=-2.0)
    assert torch.equal(c, torch.full_like(c, 10.5 - 42.0))
    # identity on the B side returns A: a transposed operand or a swapped leading dimension cannot pass
    x, _, _ = testing.make_float_case(128, 64, 64, seed=2, device='cuda')
    eye = torch.eye(64, device='cuda').t()
    out = torch.zeros(128, 64, device='cuda')
    yan.gemm_float_nt(x, eye, out)
    assert torch.equal(out, x)
    # k == 0: c <- beta * c
    out2 = out.clone()
    yan.gemm_float_nt(torch.zeros(0, 128, device='cuda').t(), torch.zeros(0, 64, device='cuda').t(), out2, alpha=1.0, beta=3.0)
    assert torch.equal(out2, 3.0 * out)
    # tests/test_simple.py:35 times the kernel whose name contains 'gemm_cute'
    big = testing.make_float_case(4096, 4096, 1024, seed=3, device='cuda')
    t = yan.bench_kineto(lambda: yan.gemm_float_nt(*big), 'gemm_cute', suppress_kineto_output=True)
    assert 0 < t < 5e-3


def test_float_golden_fixture(repo_root):
    """The committed fp32 fixture: raw buffers with padded leading dimensions through the C entry, and the
    exact-integer case through the JIT entry, bit for bit."""
    z = np.load(os.path.join(repo_root, 'tests', 'golden', 'float_small.npz'))
    m, n, k, lda, ldb, ldc = (int(v) for v in z['dims'])
    alpha, beta = (float(v) for v in z['alpha_beta'])
    da, db, dc = (torch.from_numpy(z[name]).cuda() for name in ('a_buf', 'b_buf', 'c_buf'))
    assert capi.load().yan_gemm_float_nt(m, n, k, alpha, da.data_ptr(), lda, db.data_ptr(), ldb, beta, dc.data_ptr(), ldc, None) == 0
    got = dc.cpu().numpy().astype(np.float64)
    assert oracle.calc_diff(got[:, :n], z['expected_f64']) < FLOAT_TOL and _float_close(got[:, :n], z['expected_f64'], k)
    assert np.array_equal(got[:, n:], z['c_buf'][:, n:].astype(np.float64))
    a, b, c = torch.from_numpy(z['int_a']).cuda().t(), torch.from_numpy(z['int_b']).cuda().t(), torch.from_numpy(z['int_c']).cuda()
    ia, ib = (float(v) for v in z['int_alpha_beta'])
    yan.gemm_float_nt(a, b, c, alpha=ia, beta=ib)
    assert np.array_equal(c.cpu().numpy().astype(np.float64), z['int_expected'])


@pytest.mark.parametrize('m,n,k,lda,ldb,ldc', [(132, 68, 37, 140, 72, 80), (4, 4, 1, 4, 4, 4), (260, 516, 129, 260, 516, 516),
                                               (128, 64, 16, 128, 64, 64), (1024, 2112, 300, 1032, 2112, 2116)])
def test_capi_float_matches_raw_buffer_oracle(m, n, k, lda, ldb, ldc):
    """The C entry on raw buffers with leading dimensions, any m and n that are multiples of 4: against the C triple
    loop that indexes A[i + t*lda], B[j + t*ldb], C[i*ldc + j]; what lies outside the m x n window is left alone."""
    from oracle import c_oracle
    _announce('capi fp32', m, n, k, lda, ldb, ldc)
    g = torch.Generator().manual_seed(11)
    a_buf, b_buf = torch.randn(k, lda, generator=g), torch.randn(k, ldb, generator=g)
    c_buf = torch.randn(m, ldc, generator=g)
    da, db, dc = a_buf.cuda(), b_buf.cuda(), c_buf.cuda()
    lib = capi.load()
    for alpha, beta in ((1.0, 0.0), (0.75, -1.5)):
        dc.copy_(c_buf)
        assert lib.yan_gemm_float_nt(m, n, k, alpha, da.data_ptr(), lda, db.data_ptr(), ldb, beta, dc.data_ptr(), ldc, None) == 0
        got = dc.cpu().numpy().astype(np.float64)
        want = c_oracle.gemm_float_nt(m, n, k, alpha, a_buf.numpy(), lda, b_buf.numpy(), ldb, beta, c_buf.numpy(), ldc).reshape(m, ldc)
        assert _float_close(got[:, :n], want[:, :n], k) and oracle.calc_diff(got[:, :n], want[:, :n]) < FLOAT_TOL
        assert np.array_equal(got[:, n:], c_buf.numpy()[:, n:].astype(np.float64))
    if m % 128 == 0 and n % 64 == 0 and lda == m and ldb == n and ldc == n:
        a, b = da.t()[:m], db.t()[:n]
        via_jit, via_lib = torch.zeros(m, n, device='cuda'), torch.zeros(m, n, device='cuda')
        yan.gemm_float_nt(a, b, via_jit)
        assert capi.gemm_float_nt(a, b, via_lib) == 0
        assert torch.equal(via_jit, via_lib)            # same kernel source, same tile choice: same bits


@pytest.mark.parametrize('m,n,k', [s for s in testing.FP8_TEST_SHAPES if s[0] * s[1] * s[2] <= 7e10])
@pytest.mark.parametrize('col_major', [False, True])
def test_fp8_parity_vs_oracle(m, n, k, col_major):
    _announce('fp8', m, n, k, 'col-major scales' if col_major else 'row-major scales')
    (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=42, device='cuda', col_major_scales=col_major)
    out.fill_(float('nan'))
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
    torch.cuda.synchronize()
    got = _np(out)
    assert np.isfinite(got).all()
    ref = _fp8_ref(a8, sa, b8, sb)
    assert oracle.calc_diff(got, ref) < FP8_TOL
    # far tighter than the contract: only the bf16 output rounding and fp32 summation order separate the two
    assert oracle.calc_diff(got, ref) < 1e-5
    # element-wise: within one bf16 step of the fp32 value, plus the matrix core's own summation error. The fp8
    # MFMA does not carry full fp32 precision inside a 128-deep block: measured errors reach about 2^-15 of the
    # largest product in the block, i.e. ~1e-5 of max|out| on N(0,1) data (this is why blocks are folded in fp32).
    assert bool(np.all(np.abs(got - ref) <= np.abs(ref) * 2.0 ** -7 + 1e-4 * np.abs(ref).max()))


def test_fp8_golden_fixtures(repo_root):
    z = np.load(os.path.join(repo_root, 'tests', 'golden', 'gemm_small.npz'))

    def dev(codes):
        return torch.from_numpy(codes).cuda().view(torch.float8_e4m3fn)

    out = torch.zeros(64, 256, dtype=torch.bfloat16, device='cuda')
    yan.gemm_fp8_fp8_bf16_nt((dev(z['fp8_lhs']), torch.from_numpy(z['fp8_lhs_scales']).cuda()),
                             (dev(z['fp8_rhs']), torch.from_numpy(z['fp8_rhs_scales']).cuda()), out)
    assert oracle.calc_diff(_np(out), z['fp8_expected_f64']) < 1e-5
    # integer-valued operands with power-of-two scales: every partial sum is exact, so the result is too
    out = torch.zeros(40, 192, dtype=torch.bfloat16, device='cuda')
    yan.gemm_fp8_fp8_bf16_nt((dev(z['int_lhs']), torch.from_numpy(z['int_lhs_scales']).cuda()),
                             (dev(z['int_rhs']), torch.from_numpy(z['int_rhs_scales']).cuda()), out)
    assert np.array_equal(_np(out), oracle.bf16_round(z['int_expected']))


def test_grouped_and_cast_golden_fixtures(repo_root):
    """Committed fixtures for the quantisers (bit for bit) and for both grouped layouts (integer-valued operands
    with power-of-two scales: exact, so bit for bit as well; rows that must not be written keep the sentinel)."""
    z = np.load(os.path.join(repo_root, 'tests', 'golden', 'grouped_cast_small.npz'))

    def dev(codes):
        return torch.from_numpy(codes).cuda().view(torch.float8_e4m3fn)

    src = torch.from_numpy(z['cast_src_bf16_bits'].astype(np.int16)).view(torch.bfloat16).cuda()
    q, sc = yan.per_token_cast_to_fp8(src)
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), z['per_token_codes']) and np.array_equal(sc.cpu().numpy(), z['per_token_scales'])
    q, sc = yan.per_block_cast_to_fp8(src)
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), z['per_block_codes']) and np.array_equal(sc.cpu().numpy(), z['per_block_scales'])

    rhs = (dev(z['grouped_rhs']), torch.from_numpy(z['grouped_rhs_scales']).cuda())
    idx = torch.from_numpy(z['contiguous_m_indices']).cuda()
    out = torch.full((384, 192), -7.0, dtype=torch.bfloat16, device='cuda')
    yan.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((dev(z['contiguous_lhs']), torch.from_numpy(z['contiguous_lhs_scales']).cuda()), rhs, out, idx)
    want = oracle.bf16_round(z['contiguous_expected'])
    want[z['contiguous_m_indices'] < 0] = -7.0
    assert np.array_equal(_np(out), want)
    out = torch.full((2, 40, 192), -7.0, dtype=torch.bfloat16, device='cuda')
    yan.m_grouped_gemm_fp8_fp8_bf16_nt_masked((dev(z['masked_lhs']), torch.from_numpy(z['masked_lhs_scales']).cuda()), rhs, out,
                                              torch.from_numpy(z['masked_m']).cuda(), 40)
    want = oracle.bf16_round(z['masked_expected'])
    want[1, 7:] = -7.0
    assert np.array_equal(_np(out), want)


def test_fp8_exact_cases_and_scale_indexing():
    rng = np.random.default_rng(12)
    m, n, k = 130, 448, 640          # ragged m, n = 3.5 scale blocks, 5 K blocks
    va = rng.integers(-2, 3, size=(m, k)).astype(np.float32)
    vb = rng.integers(-2, 3, size=(n, k)).astype(np.float32)
    a8 = torch.from_numpy(oracle.e4m3fn_encode(va)).cuda().view(torch.float8_e4m3fn)
    b8 = torch.from_numpy(oracle.e4m3fn_encode(vb)).cuda().view(torch.float8_e4m3fn)
    sa = (2.0 ** rng.integers(-3, 4, size=(m, 5))).astype(np.float32)
    sb = (2.0 ** rng.integers(-3, 4, size=(4, 5))).astype(np.float32)
    out = torch.zeros(m, n, dtype=torch.bfloat16, device='cuda')
    yan.gemm_fp8_fp8_bf16_nt((a8, torch.from_numpy(sa).cuda()), (b8, torch.from_numpy(sb).cuda()), out)
    want = oracle.gemm_fp8_block_scaled_ref(oracle.e4m3fn_encode(va), sa, oracle.e4m3fn_encode(vb), sb)
    assert np.array_equal(_np(out), oracle.bf16_round(want))
    # one non-zero K block with arbitrary scales isolates sA[m, kb] and sB[n // 128, kb]
    kb = 3
    a0 = np.zeros_like(va)
    a0[:, kb * 128:(kb + 1) * 128] = va[:, kb * 128:(kb + 1) * 128]
    sa_r = (rng.random((m, 5)) + 0.5).astype(np.float32)
    sb_r = (rng.random((4, 5)) + 0.5).astype(np.float32)
    a08 = torch.from_numpy(oracle.e4m3fn_encode(a0)).cuda().view(torch.float8_e4m3fn)
    yan.gemm_fp8_fp8_bf16_nt((a08, torch.from_numpy(sa_r).cuda()), (b8, torch.from_numpy(sb_r).cuda()), out)
    part = va[:, kb * 128:(kb + 1) * 128].astype(np.float64) @ vb[:, kb * 128:(kb + 1) * 128].astype(np.float64).T
    want = part * sa_r[:, kb].astype(np.float64)[:, None] * np.repeat(sb_r[:, kb].astype(np.float64), 128)[:n][None, :]
    assert bool(np.all(np.abs(_np(out) - want) <= np.abs(want) * 2.0 ** -7 + 1e-6))


def test_fp8_linearity_and_layout_independence_at_headline_size():
    """cfg3 (4096 x 7168 x 7168): doubling every activation scale doubles the output exactly; row-major and
    token-contiguous scale tensors give identical bits; sampled rows match the oracle; the full matrix matches a
    chunked fp32 matmul of the dequantised operands on the device."""
    m, n, k = testing.BASELINE_FP8['cfg3']
    _announce('fp8 cfg3', m, n, k)
    (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=42, device='cuda', gen_device='cuda')
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
    out2 = torch.zeros_like(out)
    yan.gemm_fp8_fp8_bf16_nt((a8, yan.get_col_major_tensor(sa * 2)), (b8, sb), out2)
    assert torch.equal(out2.float(), out.float() * 2)
    rows = np.random.default_rng(1).choice(m, 48, replace=False)
    ref = _fp8_ref(a8[rows], sa[rows], b8, sb)
    assert oracle.calc_diff(_np(out[rows]), ref) < 1e-5
    wd = testing.dequant_rhs(b8, sb)
    num = den = 0.0
    for r0 in range(0, m, 1024):
        ref = testing.dequant_lhs(a8[r0:r0 + 1024], sa[r0:r0 + 1024]) @ wd.t()
        got = out[r0:r0 + 1024].float()
        num += (got.double() * ref.double()).sum().item()
        den += (got.double() ** 2 + ref.double() ** 2).sum().item()
    assert 1 - 2 * num / den < FP8_TOL


def test_fp8_decode_shape():
    m, n, k = testing.BASELINE_FP8['cfg4']
    _announce('fp8 cfg4', m, n, k)
    (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=42, device='cuda')
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
    assert oracle.calc_diff(_np(out), _fp8_ref(a8, sa, b8, sb)) < 1e-5


def test_fp8_decode_shapes_are_repeatable():
    """The decode shapes (tiled kernel on narrow tiles with a ring of LDS stages; weight-streaming kernel up to 16
    rows) keep no state between calls: repeated and interleaved calls give the same bits."""
    (a8, sa), (b8, sb), out = testing.make_fp8_case(64, 4096, 7168, seed=3, device='cuda')
    (c8, sc), (d8, sd), out_small = testing.make_fp8_case(40, 2112, 640, seed=4, device='cuda')
    (e8, se), (f8, sf), out_one = testing.make_fp8_case(1, 4096, 7168, seed=5, device='cuda')
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
    yan.gemm_fp8_fp8_bf16_nt((e8, se), (f8, sf), out_one)
    first, first_one = out.clone(), out_one.clone()
    ref_small = _fp8_ref(c8, sc, d8, sd)
    for _ in range(5):
        out.fill_(float('nan'))
        out_one.fill_(float('nan'))
        yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
        yan.gemm_fp8_fp8_bf16_nt((c8, sc), (d8, sd), out_small)
        yan.gemm_fp8_fp8_bf16_nt((e8, se), (f8, sf), out_one)
        assert torch.equal(out, first) and torch.equal(out_one, first_one)
        assert oracle.calc_diff(_np(out_small), ref_small) < 1e-5
    assert oracle.calc_diff(_np(first), _fp8_ref(a8, sa, b8, sb)) < 1e-5
    assert oracle.calc_diff(_np(first_one), _fp8_ref(e8, se, f8, sf)) < 1e-5


@pytest.mark.parametrize('m,n,k', testing.FP8_SPLIT_K_SHAPES)
@pytest.mark.parametrize('col_major', [False, True])
def test_split_k_parity_vs_oracle(m, n, k, col_major):
    """Problems whose K the entry point splits over 2 to 4 workgroups per tile (every ring tile, every factor, ragged edges,
    K ranges of unequal length): parity against the oracle to the bar of the unsplit kernel, the same bits from the
    library's split-K entry point, which writes nothing past row m, and arrival counters back at zero."""
    plan = yan.gemm.fp8_split_k_plan(m, n, k, yan.get_num_sms(), col_major)
    assert plan is not None and (plan[1]['BLOCK_M'], plan[1]['BLOCK_N'], plan[1]['SPLIT_K']) == testing.FP8_SPLIT_K_PLAN_OF_SHAPE[(m, n, k)]
    _announce('fp8 split-k', m, n, k, plan[1]['BLOCK_M'], plan[1]['BLOCK_N'], plan[1]['SPLIT_K'], 'col-major' if col_major else 'row-major')
    (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=42, device='cuda', col_major_scales=col_major)
    out.fill_(float('nan'))
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
    torch.cuda.synchronize()
    got, ref = _np(out), _fp8_ref(a8, sa, b8, sb)
    assert np.isfinite(got).all()
    assert oracle.calc_diff(got, ref) < 1e-5
    assert bool(np.all(np.abs(got - ref) <= np.abs(ref) * 2.0 ** -7 + 1e-4 * np.abs(ref).max()))
    workspace = capi.split_k_workspace()
    padded = torch.full((m + 3, n), 7.0, dtype=torch.bfloat16, device='cuda')
    assert capi.gemm_fp8_fp8_bf16_nt_split_k((a8, sa), (b8, sb), padded, workspace) == 0
    torch.cuda.synchronize()
    assert torch.equal(padded[:m], out) and bool((padded[m:] == 7.0).all())
    counters = capi.load().yan_gemm_split_k_counter_bytes()
    assert int(workspace[:counters].view(torch.int32).abs().sum()) == 0


def test_split_k_launches_of_different_shapes_share_a_workspace():
    """One workspace per stream serves every split-K launch on it: shapes with different tiles and factors interleaved,
    the caches flushed between some rounds so that the parts arrive in another order, give the same bits every time (the
    part that arrives last adds the parts up in the order of their K ranges, whichever it is)."""
    shapes = [(64, 4096, 7168), (33, 2112, 5376), (300, 4100, 6144), (129, 2112, 7168), (17, 3076, 6272)]
    cases = [testing.make_fp8_case(*shape, seed=5 + i, device='cuda', gen_device='cuda') for i, shape in enumerate(shapes)]
    dense_shapes = [(64, 4096, 7168), (200, 4100, 3080), (129, 2112, 5120)]        # the dense split-K kernels share it too
    dense_cases = [testing.make_bf16_case(*shape, seed=15 + i, scale=shape[2] ** -0.5, device='cuda', gen_device='cuda') for i, shape in enumerate(dense_shapes)]
    firsts, dense_firsts = [], []
    for (lhs, rhs, out) in cases:
        yan.gemm_fp8_fp8_bf16_nt(lhs, rhs, out)
        firsts.append(out.clone())
    for (a, b, c) in dense_cases:
        yan.gemm_bf16_tn(a, b, c)
        dense_firsts.append(c.clone())
    for ((a8, sa), (b8, sb), out), first in zip(cases, firsts):
        assert float(yan.calc_diff(first.float(), testing.dequant_lhs(a8, sa) @ testing.dequant_rhs(b8, sb).t())) < 1e-5
    for (a, b, c), first in zip(dense_cases, dense_firsts):
        assert float(yan.calc_diff(first.float(), a.float() @ b.float().t())) < 1e-5
    flush = torch.empty(512 << 18, dtype=torch.int, device='cuda')
    for it in range(12):
        if it % 3 == 0:
            flush.zero_()
        for i, (lhs, rhs, out) in enumerate(cases):
            out.fill_(float('nan'))
            yan.gemm_fp8_fp8_bf16_nt(lhs, rhs, out)
            if i < len(dense_cases):
                a, b, c = dense_cases[i]
                c.fill_(float('nan'))
                yan.gemm_bf16_tn(a, b, c)
        for (_, _, out), first in zip(cases, firsts):
            assert torch.equal(out, first), it
        for (_, _, c), first in zip(dense_cases, dense_firsts):
            assert torch.equal(c, first), it


def test_split_k_entry_point_checks_its_workspace():
    """A workspace smaller than the plan needs, or none, is an error and launches nothing; problems whose K is not split
    do not look at it."""
    (a8, sa), (b8, sb), out = testing.make_fp8_case(64, 4096, 7168, seed=1, device='cuda', gen_device='cuda')
    out.fill_(3.0)
    small = torch.zeros(1 << 20, dtype=torch.uint8, device='cuda')
    assert capi.gemm_fp8_fp8_bf16_nt_split_k((a8, sa), (b8, sb), out, small) == 1          # hipErrorInvalidValue
    lib = capi.load()
    assert lib.yan_gemm_fp8_fp8_bf16_nt_split_k(a8.data_ptr(), sa.data_ptr(), sa.stride(0), sa.stride(1), b8.data_ptr(), sb.data_ptr(),
                                                out.data_ptr(), 64, 4096, 7168, None, 0, None, 1 << 30) == 1
    torch.cuda.synchronize()
    assert bool((out == 3.0).all())
    (c8, sc), (d8, sd), out2 = testing.make_fp8_case(300, 96, 640, seed=2, device='cuda')
    assert capi.select_split_k(300, 96, 640, yan.get_num_sms()) is None
    assert capi.gemm_fp8_fp8_bf16_nt_split_k((c8, sc), (d8, sd), out2, small) == 0
    plain = torch.zeros_like(out2)
    assert capi.gemm_fp8_fp8_bf16_nt((c8, sc), (d8, sd), plain) == 0
    assert torch.equal(out2, plain)


@pytest.mark.parametrize('m,n,k', [(128, 4096, 7168), (512, 4096, 2048), (1024, 7168, 1024)])
def test_ring_of_stages_is_race_free(m, n, k):
    """Tiles below 256 x 256 keep several k-tiles in flight in a ring of LDS stages, synchronised by counting the
    wave's outstanding copies. A slip there would show as run-to-run differences: 30 launches, cache flushed between
    some of them so that the copies land in a different order, must give the same bits, FP8 and bf16."""
    (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=11, device='cuda', gen_device='cuda')
    a, b, c = testing.make_bf16_case(m, n, k, seed=12, scale=k ** -0.5, device='cuda', gen_device='cuda')
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
    yan.gemm_bf16_tn(a, b, c)
    first8, first16 = out.clone(), c.clone()
    assert float(yan.calc_diff(first8.float(), testing.dequant_lhs(a8, sa) @ testing.dequant_rhs(b8, sb).t())) < 1e-3
    assert float(yan.calc_diff(first16.float(), a.float() @ b.float().t())) < 1e-5
    flush = torch.empty(512 << 18, dtype=torch.int, device='cuda')
    for it in range(30):
        if it % 3 == 0:
            flush.zero_()
        out.fill_(float('nan'))
        c.fill_(float('nan'))
        yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
        yan.gemm_bf16_tn(a, b, c)
        assert torch.equal(out, first8) and torch.equal(c, first16), it


def test_fp8_outlier_16384_cubed():
    """cfg5: uniform[-4,4] sources with 1% of entries x50. Sampled rows against the oracle, plus finiteness."""
    m, n, k = testing.BASELINE_FP8['cfg5']
    _announce('fp8 cfg5', m, n, k)
    (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=42, dist='outlier', device='cuda', gen_device='cuda')
    assert not torch.isnan(a8.view(torch.uint8).float()).any()
    assert int((a8.view(torch.uint8) & 0x7F).max()) <= 0x7E and int((b8.view(torch.uint8) & 0x7F).max()) <= 0x7E
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
    torch.cuda.synchronize()
    rows = np.random.default_rng(2).choice(m, 32, replace=False)
    ref = _fp8_ref(a8[rows], sa[rows], b8, sb)
    got = _np(out[rows])
    assert np.isfinite(got).all()
    assert oracle.calc_diff(got, ref) < FP8_TOL
    assert oracle.calc_diff(got, ref) < 1e-5
    assert bool(torch.isfinite(out[::97].float()).all())
    # the whole 16384 x 16384 output (4096 tiles) against a chunked fp32 matmul of the dequantised operands on the device:
    # over everything, and slab by slab so that no band of tiles can hide behind the rest
    wd = testing.dequant_rhs(b8, sb)
    num = den = 0.0
    for r0 in range(0, m, 1024):
        ref = testing.dequant_lhs(a8[r0:r0 + 1024], sa[r0:r0 + 1024]) @ wd.t()
        got = out[r0:r0 + 1024].float()
        assert bool(torch.isfinite(got).all())
        slab_num = (got.double() * ref.double()).sum().item()
        slab_den = (got.double() ** 2 + ref.double() ** 2).sum().item()
        assert 1 - 2 * slab_num / slab_den < 1e-4, r0
        num, den = num + slab_num, den + slab_den
    assert 1 - 2 * num / den < 1e-4


# ----------------------------------------------------------------------------- the compute-unit cap (num_sms)
def _event_ms(fn, reps):
    fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) / reps


@pytest.mark.parametrize('m,n,k', testing.CAPPED_SHAPES)
def test_num_sms_caps_the_workgroups_without_changing_a_bit(m, n, k):
    """The reference's persistent kernels launch `num_sms` blocks (yan/include/gemm/fp8_gemm.cuh:40,
    yan/jit_kernels/gemm.py:26-30, utils.py:6-29). Here a cap below the device's compute units launches that many
    workgroups (a multiple of 8), each walking several tiles: same kernel, same tile, same bits as one workgroup per
    tile; and through set_num_sms the public entries stay within tolerance of the oracle."""
    from yan_amd.jit_kernels import bf16_gemm, gemm
    _announce('num_sms cap', m, n, k)
    cap, stream = testing.NUM_SMS_CAP, torch.cuda.current_stream()
    full = yan.get_num_sms()
    assert cap < full
    (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=21, device='cuda')
    name, keys, defs, smem, tmpl = gemm.fp8_kernel_plan(m, n, k, full, False)
    rt = jit.build(name, defs, jit.generate(gemm.includes, defs, jit.cpp_format(tmpl, keys)))
    capped = torch.full_like(out, float('nan'))
    assert rt(a8, sa, b8, sb, out, m, stream, full, smem, sa.stride(0), sa.stride(1)) == 0
    assert rt(a8, sa, b8, sb, capped, m, stream, cap, smem, sa.stride(0), sa.stride(1)) == 0
    assert torch.equal(capped, out)
    assert oracle.calc_diff(_np(out), _fp8_ref(a8, sa, b8, sb)) < 1e-5
    a, b, c = testing.make_bf16_case(m, n, k, seed=22, device='cuda')
    results = []
    for num_sms_cap in (0, cap):
        name, dkeys, ddefs = bf16_gemm.dense_kernel_plan(m, n, k, torch.bfloat16, full, num_sms_cap)
        drt = jit.build(name, ddefs, jit.generate(bf16_gemm.includes, ddefs, jit.cpp_format(bf16_gemm.template, dkeys)))
        c = torch.full_like(c, float('nan'))
        assert drt(m, n, k, a, b, c, stream) == 0
        results.append(c)
    assert torch.equal(results[0], results[1])
    try:
        yan.set_num_sms(cap)
        assert yan.get_num_sms() == cap
        out2, c2 = torch.full_like(out, float('nan')), torch.full_like(c, float('nan'))
        yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out2)
        yan.gemm_bf16_tn(a, b, c2)
        assert torch.equal(out2, out)                 # the block-scaled sum is formed in the same order by every tile
        assert float(yan.calc_diff(c2.float(), a.float() @ b.float().t())) < BF16_TOL
    finally:
        yan.set_num_sms(full)


def test_grouped_layouts_under_a_compute_unit_cap_give_the_same_bits():
    """Both grouped layouts with `set_num_sms(64)`: 64 workgroups walk the slots, several tiles each (for the contiguous
    layout on 256-row tiles the slots of `ContiguousSlots`, two-group rows first), and write the bits of the uncapped
    launch."""
    from yan_amd.jit_kernels.m_grouped_gemm import grouped_kernel_plan
    cap, full = testing.NUM_SMS_CAP, yan.get_num_sms()
    rows, n, k, pad_blocks = testing.GROUPED_TWO_GROUP_ROWS_FIRST_CASE
    _announce('grouped contiguous under a cap', rows, n, k, cap)
    (a8, sa), (b8, sb), out, idx = testing.make_grouped_contiguous_case(rows, n, k, seed=5, padding_blocks=pad_blocks)
    a8, sa, b8, sb, idx = a8.cuda(), sa.cuda(), b8.cuda(), sb.cuda(), idx.cuda()
    assert grouped_kernel_plan('GroupedContiguous', len(rows), a8.size(0), n, k, cap)[1]['BLOCK_M'] == 256
    groups, m_max, n2, k2, masked, expected_m = testing.GROUPED_MASKED_TEST_CASES[6]
    (x8, sx), (w8, sw), out2, mm = testing.make_grouped_masked_case(groups, m_max, n2, k2, masked, seed=6)
    x8, sx, w8, sw, mm = x8.cuda(), sx.cuda(), w8.cuda(), sw.cuda(), mm.cuda()
    results = {}
    try:
        for cus in (full, cap):
            yan.set_num_sms(cus)
            got, got2 = out.cuda(), out2.cuda()
            yan.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((a8, sa), (b8, sb), got, idx)
            _announce('grouped masked under a cap', groups, m_max, n2, k2, cus)
            yan.m_grouped_gemm_fp8_fp8_bf16_nt_masked((x8, sx), (w8, sw), got2, mm, expected_m)
            torch.cuda.synchronize()
            results[cus] = (got, got2)
    finally:
        yan.set_num_sms(full)
    assert torch.equal(results[cap][0], results[full][0])
    assert torch.equal(results[cap][1], results[full][1])
    assert bool((results[full][0][idx >= 0] != -7.0).any())


@pytest.mark.parametrize('cap', testing.ODD_CAP_CASE[1])
def test_walks_under_a_cap_that_is_no_multiple_of_the_xcds_reach_every_tile(cap):
    """18 tiles of 256 x 256 leave an empty slot at the end of six of the eight XCDs' ranges; 3 or 5 persistent workgroups
    walk across those ranges and must not stop at the first empty slot. Both persistent kernels, against their own
    uncapped launch (same bits: a tile's sum does not depend on which workgroup runs it) and the oracle."""
    (m, n, k), _ = testing.ODD_CAP_CASE
    _announce('odd num_sms cap', cap, m, n, k)
    stream = torch.cuda.current_stream()
    (fp8_name, fp8_keys, fp8_defs, fp8_inc, fp8_tmpl), _ = testing.odd_cap_plans(cap)
    rt = jit.build(fp8_name, fp8_defs, jit.generate(fp8_inc, fp8_defs, jit.cpp_format(fp8_tmpl, fp8_keys)))
    (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=23, device='cuda', col_major_scales=True)
    capped = torch.full_like(out, float('nan'))
    assert rt(a8, sa, b8, sb, out, m, stream, yan.get_num_sms(), 0) == 0
    assert rt(a8, sa, b8, sb, capped, m, stream, cap, 0) == 0
    assert torch.equal(capped, out)
    assert oracle.calc_diff(_np(out), _fp8_ref(a8, sa, b8, sb)) < 1e-5
    a, b, c = testing.make_bf16_case(m, n, k, seed=24, device='cuda')
    results = []
    for this_cap in (0, cap):
        _, (name, keys, defs, inc, tmpl) = testing.odd_cap_plans(this_cap)
        drt = jit.build(name, defs, jit.generate(inc, defs, jit.cpp_format(tmpl, keys)))
        c = torch.full_like(c, float('nan'))
        assert drt(m, n, k, a, b, c, stream) == 0
        results.append(c)
    assert torch.equal(results[0], results[1])
    assert oracle.calc_diff(_np(results[1]), oracle.gemm_bf16_tn_ref(_np(a), _np(b))) < BF16_TOL


def test_num_sms_cap_is_what_runs_at_the_headline_size():
    """cfg3 under a cap of 64 of 256 compute units: identical bits, and two to four times the time, i.e. the cap is the
    number of compute units that work (448 tiles: 7 rounds of 64 instead of 1.75 rounds of 256). Less than four times:
    a quarter of the chip is not power-limited and each of its compute units runs a tile about a third faster."""
    from yan_amd.jit_kernels import gemm
    m, n, k = testing.BASELINE_FP8['cfg3']
    _announce('num_sms cap at cfg3', m, n, k)
    (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=42, device='cuda', gen_device='cuda', col_major_scales=True)
    full, stream = yan.get_num_sms(), torch.cuda.current_stream()
    name, keys, defs, smem, tmpl = gemm.fp8_kernel_plan(m, n, k, full, True)
    rt = jit.build(name, defs, jit.generate(gemm.includes, defs, jit.cpp_format(tmpl, keys)))
    capped = torch.full_like(out, float('nan'))
    t_full = _event_ms(lambda: rt(a8, sa, b8, sb, out, m, stream, full, smem), 20)
    t_cap = _event_ms(lambda: rt(a8, sa, b8, sb, capped, m, stream, 64, smem), 10)
    assert torch.equal(capped, out)
    assert 1.7 * t_full < t_cap < 6.0 * t_full, (t_full, t_cap)


# ----------------------------------------------------------------------------- the ahead-of-time C-ABI library
def test_tuner_times_a_space_of_tiles_on_the_device():
    """The empirical half of compile_and_tune (yan/jit_kernels/tuner.py:24-69): every candidate of `space` is built, run
    once, timed over back-to-back launches after a cache flush, and the fastest is kept and memoised."""
    from yan_amd.jit_kernels import bf16_gemm
    from yan_amd.jit_kernels.tuner import JITTuner
    m = n = k = 1024
    a, b, c = testing.make_bf16_case(m, n, k, seed=3, device='cuda')
    args = (m, n, k, a, b, c, torch.cuda.current_stream())
    from yan_amd.jit_kernels.heuristics import get_dense_num_stages
    space = tuple({'BLOCK_M': bm, 'BLOCK_N': bn, 'NUM_STAGES': get_dense_num_stages(bm, bn), 'NUM_SMS': 0} for bm, bn in ((256, 256), (128, 128), (64, 64)))
    tuner = JITTuner()
    kw = dict(name='gemm_bf16_tn', keys={}, space=space, includes=bf16_gemm.includes,
              arg_defs=bf16_gemm._arg_defs(torch.bfloat16), template=bf16_gemm.template, args=args)
    best = tuner.compile_and_tune(**kw)
    assert tuner.compile_and_tune(**kw) is best                       # memoised
    chosen = list(tuner.tuned_keys.values())[0]
    assert (chosen['BLOCK_M'], chosen['BLOCK_N']) in ((256, 256), (128, 128), (64, 64))
    c.zero_()
    assert best(*args) == 0
    assert float(yan.calc_diff(c.float(), a.float() @ b.float().t())) < 1e-5


@pytest.mark.parametrize('m,n,k', testing.TUNED_SHAPES)
def test_entry_points_pick_the_fastest_of_three_tiles_when_asked(m, n, k, monkeypatch):
    """With YAN_TUNE_TILES=1 the first call of a shape hands the cost model's three best tiles to the tuner
    (yan/jit_kernels/cute_gemm.py:42-53, tuner.py:42-69); the winner is memoised per shape and the result is the same
    GEMM."""
    from yan_amd.jit_kernels import bf16_gemm, gemm
    from yan_amd.jit_kernels.tuner import jit_tuner
    _announce('tuned tiles', m, n, k)
    monkeypatch.setenv('YAN_TUNE_TILES', '1')
    a, b, c = testing.make_bf16_case(m, n, k, seed=5, scale=k ** -0.5, device='cuda', gen_device='cuda')
    yan.gemm_bf16_tn(a, b, c)
    name, keys, space, _ = bf16_gemm.dense_tuning_plan(m, n, k, torch.bfloat16, yan.get_num_sms(), 0)
    chosen = jit_tuner.tuned_keys[(name, str({key: keys[key] for key in sorted(keys)}))]
    assert chosen in list(space) and len(space) == 3
    pick = torch.randperm(m, device='cuda')[:512]
    assert float(yan.calc_diff(c[pick].float(), a[pick].float() @ b.float().t())) < BF16_TOL
    (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=6, device='cuda', gen_device='cuda', col_major_scales=True)
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
    name, keys, space, _, _ = gemm.fp8_tuning_plan(m, n, k, yan.get_num_sms(), True)
    chosen = jit_tuner.tuned_keys[(name, str({key: keys[key] for key in sorted(keys)}))]
    assert chosen in list(space) and len(space) == 3
    ref = testing.dequant_lhs(a8[pick], sa[pick]) @ testing.dequant_rhs(b8, sb).t()
    assert float(yan.calc_diff(out[pick].float(), ref)) < 1e-5
    # the tile the cost model alone would have picked gives the same bits (every tile sums the K blocks in the same order)
    monkeypatch.setenv('YAN_TUNE_TILES', '0')
    again = torch.zeros_like(out)
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), again)
    assert torch.equal(again, out)


@pytest.mark.parametrize('block_m,block_n,shape', testing.FP8_EXPLICIT_TILE_CASES)
def test_fp8_tiles_whose_slabs_straddle_weight_scale_blocks(block_m, block_n, shape):
    """256 x 224, 256 x 192 and 64 x 160 tiles, built through the reference's keys (yan/jit_kernels/gemm.py:9-16): wave
    slabs of 112, 96 and 80 columns cross the boundaries of the 128-wide weight-scale blocks and do not divide the 64
    lanes of the row stores. Same bits as the tile the cost model picks (every tile sums the K blocks in the same order), parity against
    the oracle, ragged edges left alone."""
    from yan_amd import jit
    m, n, k = shape
    _announce('explicit fp8 tile', block_m, block_n, m, n, k)
    (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=11, device='cuda', col_major_scales=True)
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
    name, keys, arg_defs, code_template = testing.fp8_explicit_tile_plan(block_m, block_n, n, k)
    runtime = jit.build(name, arg_defs, jit.generate(yan.gemm.includes, arg_defs, jit.cpp_format(code_template, keys)))
    padded = torch.full((m + 3, n), 7.0, dtype=torch.bfloat16, device='cuda')
    rc = runtime(a8, sa, b8, sb, padded, m, torch.cuda.current_stream(), yan.get_num_sms(), 0)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(padded[:m], out) and bool((padded[m:] == 7.0).all())
    assert oracle.calc_diff(_np(out), _fp8_ref(a8, sa, b8, sb)) < 1e-5


# ----------------------------------------------------------------------------- quantisers in front of the FP8 GEMM
def _oracle_per_token(x):
    q, s_ = oracle.per_token_cast_to_fp8(x.float().numpy())
    return torch.from_numpy(q), torch.from_numpy(s_)


def _oracle_per_block(w):
    q, s_ = oracle.per_block_cast_to_fp8(w.float().numpy())
    return torch.from_numpy(q), torch.from_numpy(s_)


def _tie_rows():
    """Rows of 128 values with |max| = 448 exactly (so the quantiser's factor is 1.0) holding every positive e4m3
    value, every midpoint between neighbours and the fp32 numbers just below and above each midpoint, both signs:
    any deviation from round-to-nearest-even, or from exact handling of subnormals, changes a code."""
    vals = np.sort(np.unique(np.abs(oracle.e4m3fn_decode_table()[np.isfinite(oracle.e4m3fn_decode_table())])))
    mids = (vals[:-1] + vals[1:]) / 2
    cand = np.concatenate([vals, mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9))]).astype(np.float32)
    cand = np.concatenate([cand, -cand])
    rows = -(-cand.size // 127)
    buf = np.zeros((rows, 128), dtype=np.float32)
    buf[:, 0] = 448.0
    flat = np.zeros(rows * 127, dtype=np.float32)
    flat[:cand.size] = cand
    buf[:, 1:] = flat.reshape(rows, 127)
    return torch.from_numpy(buf)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('m,k', [(1, 128), (63, 256), (300, 640), (4096, 7168)])
def test_per_token_cast_is_bit_identical_to_the_oracle(m, k, dtype):
    g = torch.Generator().manual_seed(m + k)
    x = (torch.randn(m, k, generator=g) * 3).to(dtype)
    x[m // 2, :128] = 0                                     # an all-zero group: amax clamps at 1e-4
    want_q, want_s = _oracle_per_token(x)
    q, sc = yan.per_token_cast_to_fp8(x.cuda())
    assert q.dtype == torch.float8_e4m3fn and q.shape == (m, k) and sc.shape == (m, k // 128)
    assert torch.equal(q.view(torch.uint8).cpu(), want_q) and torch.equal(sc.cpu(), want_s)
    # token-contiguous scales: same values, the layout get_col_major_tensor gives
    q2, sc2 = yan.per_token_cast_to_fp8(x.cuda(), col_major_scales=True)
    assert sc2.stride(0) == 1 and torch.equal(sc2.cpu(), want_s) and torch.equal(q2.view(torch.uint8), q.view(torch.uint8))
    assert yan.get_col_major_tensor(sc2).data_ptr() == sc2.data_ptr()
    # the harness quantiser (torch ops with true tensor / tensor divisions) run on the device
    tq, ts = testing.per_token_cast_to_fp8(x.cuda())
    assert torch.equal(ts, sc) and torch.equal(tq.view(torch.uint8), q.view(torch.uint8))
    # the C-ABI library gives the JIT kernel's bits
    lq, ls = torch.empty_like(q), torch.empty_like(sc)
    assert capi.per_token_cast_to_fp8(x.cuda(), lq, ls) == 0
    assert torch.equal(lq.view(torch.uint8), q.view(torch.uint8)) and torch.equal(ls, sc)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('n,k', [(128, 128), (129, 128), (300, 640), (7168, 7168)])
def test_per_block_cast_is_bit_identical_to_the_oracle(n, k, dtype):
    g = torch.Generator().manual_seed(n * 3 + k)
    w = torch.randn(n, k, generator=g).to(dtype)
    w[:128, :128] = 0                                       # an all-zero block
    want_q, want_s = _oracle_per_block(w)
    q, sc = yan.per_block_cast_to_fp8(w.cuda())
    assert q.shape == (n, k) and sc.shape == ((n + 127) // 128, k // 128)
    assert torch.equal(q.view(torch.uint8).cpu(), want_q) and torch.equal(sc.cpu(), want_s)
    lq, ls = torch.empty_like(q), torch.empty_like(sc)
    assert capi.per_block_cast_to_fp8(w.cuda(), lq, ls) == 0
    assert torch.equal(lq.view(torch.uint8), q.view(torch.uint8)) and torch.equal(ls, sc)


def test_casts_round_to_nearest_even_on_every_tie():
    x = _tie_rows()
    want = torch.from_numpy(oracle.e4m3fn_encode(x.numpy()))
    q, sc = yan.per_token_cast_to_fp8(x.cuda())
    assert torch.equal(sc.cpu(), torch.ones(x.size(0), 1))
    assert torch.equal(q.view(torch.uint8).cpu(), want)
    assert torch.equal(x.to(torch.float8_e4m3fn).view(torch.uint8), want)       # torch's CPU cast says the same
    # the per-block kernel shares the conversion; one 128 x 128 block, padded with copies of the first row
    w = x[:128] if x.size(0) >= 128 else torch.cat([x, x[:1].expand(128 - x.size(0), 128)])
    qb, sb = yan.per_block_cast_to_fp8(w.contiguous().cuda())
    assert float(sb) == 1.0 and torch.equal(qb.view(torch.uint8).cpu(), torch.from_numpy(oracle.e4m3fn_encode(w.numpy())))


def test_quantise_then_gemm_matches_the_oracle_end_to_end():
    """bf16 sources -> device quantisers -> FP8 GEMM, against the oracle's quantisers and product from the same sources."""
    m, n, k = 200, 384, 512
    g = torch.Generator().manual_seed(77)
    x, w = torch.randn(m, k, generator=g).bfloat16(), torch.randn(n, k, generator=g).bfloat16()
    lhs = yan.per_token_cast_to_fp8(x.cuda(), col_major_scales=True)
    rhs = yan.per_block_cast_to_fp8(w.cuda())
    out = torch.zeros(m, n, dtype=torch.bfloat16, device='cuda')
    yan.gemm_fp8_fp8_bf16_nt(lhs, rhs, out)
    qa, sa = oracle.per_token_cast_to_fp8(x.float().numpy())
    qb, sb = oracle.per_block_cast_to_fp8(w.float().numpy())
    ref = oracle.gemm_fp8_block_scaled_ref(qa, sa, qb, sb)
    assert oracle.calc_diff(out.float().cpu().numpy(), ref) < 1e-5
    # and the quantised product stays within the FP8 tolerance of the unquantised one
    assert oracle.calc_diff(out.float().cpu().numpy(), x.float().numpy() @ w.float().numpy().T) < 1e-3


# ----------------------------------------------------------------------------- grouped FP8 GEMMs
def _np_codes(t):
    return t.view(torch.uint8).cpu().numpy()


@pytest.mark.parametrize('rows,n,k,pad_blocks', testing.GROUPED_CONTIGUOUS_TEST_CASES)
def test_grouped_contiguous_parity(rows, n, k, pad_blocks):
    """Contiguous layout against the oracle (per-group block-scaled product, same seeded inputs generated on the
    CPU); rows of padding blocks (index -1) keep the caller's values; the C-ABI library gives the same bits as the
    JIT kernel; a single group gives the bits of the plain GEMM."""
    (a8, sa), (b8, sb), out, idx = testing.make_grouped_contiguous_case(rows, n, k, seed=5, padding_blocks=pad_blocks)
    m = a8.size(0)
    group_rows = [r for r in rows if r > 0]           # negative entries are padding blocks between groups
    if rows == testing.GROUPED_TWO_PASS_CASE[0]:
        # this case exists for the 256-row tile whose halves belong to different groups or to padding: make sure a
        # change of the cost table cannot silently move it to another tile
        from yan_amd.jit_kernels.m_grouped_gemm import grouped_kernel_plan
        assert grouped_kernel_plan('GroupedContiguous', len(group_rows), m, n, k, 256)[1]['BLOCK_M'] == 256
        blocks = idx.view(-1, 128)[:, 0]
        # halves of the 256-row tiles, as laid out here and as rotated by one block further down
        halves = torch.cat([b[:len(b) // 2 * 2].view(-1, 2) for b in (blocks, torch.roll(blocks, 1))])
        assert bool(((halves[:, 0] != halves[:, 1]) & (halves >= 0).all(1)).any())      # two groups in one tile
        assert bool(((halves[:, 0] < 0) & (halves[:, 1] >= 0)).any())                   # padding, then a group
        assert bool(((halves[:, 0] >= 0) & (halves[:, 1] < 0)).any())                   # a group, then padding
    if rows == testing.GROUPED_TWO_GROUP_ROWS_FIRST_CASE[0]:
        from yan_amd.jit_kernels.m_grouped_gemm import grouped_kernel_plan
        assert grouped_kernel_plan('GroupedContiguous', len(group_rows), m, n, k, 256)[1]['BLOCK_M'] == 256
        blocks = idx.view(-1, 128)[:, 0]
        halves = blocks[:len(blocks) // 2 * 2].view(-1, 2)
        two = ((halves[:, 0] != halves[:, 1]) & (halves >= 0).all(1)).nonzero().flatten()
        assert len(two) == 8 and int(two.min()) < 64 <= int(two.max()) and (m + 255) // 256 > 64
    if rows in ((512,) * 16, (384, 640) * 8):
        from yan_amd.jit_kernels.m_grouped_gemm import grouped_kernel_plan
        assert grouped_kernel_plan('GroupedContiguous', len(group_rows), m, n, k, 256)[1].get('ROWS') == 'picked on the device'
    a8d, sad, b8d, sbd, idxd = a8.cuda(), sa.cuda(), b8.cuda(), sb.cuda(), idx.cuda()
    got = out.cuda()
    assert yan.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((a8d, sad), (b8d, sbd), got, idxd) is None
    if m * n * k <= 2e10:
        ref = oracle.m_grouped_gemm_contiguous_ref(_np_codes(a8), sa.numpy(), _np_codes(b8), sb.numpy(), idx.numpy(),
                                                   out_init=out.float().numpy())
        ref = torch.from_numpy(ref)
    else:       # the per-group product on the device in fp32, rows of the oracle sampled below
        ref = out.float()
        for g in range(len(group_rows)):
            sel = (idx == g).nonzero().flatten()
            ref[sel] = (testing.dequant_lhs(a8d[sel.cuda()], sad[sel.cuda()]) @ testing.dequant_rhs(b8d[g], sbd[g]).t()).cpu()
        pick = torch.arange(0, m, 97)
        want = oracle.m_grouped_gemm_contiguous_ref(_np_codes(a8[pick]), sa[pick].numpy(), _np_codes(b8), sb.numpy(), idx[pick].numpy())
        assert oracle.calc_diff(got[pick.cuda()].float().cpu().numpy(), want) < 1e-3
    assert float(yan.calc_diff(got.float().cpu(), ref)) < 1e-3
    real = idx >= 0
    assert torch.equal(got.cpu()[~real], out[~real])                      # padding blocks untouched
    bound = ref.abs() * 2.0 ** -7 + 1e-4 * ref.abs().max()
    assert bool(((got.float().cpu() - ref).abs() <= bound)[real].all())
    via_lib = out.cuda()
    assert capi.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((a8d, sad), (b8d, sbd), via_lib, idxd) == 0
    assert torch.equal(via_lib, got)
    # scales handed over token-contiguous give the same bits
    again = out.cuda()
    yan.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((a8d, yan.get_col_major_tensor(sad)), (b8d, sbd), again, idxd)
    assert torch.equal(again, got)
    if pad_blocks:
        # the same rows rotated by one 128-row block: the padding block now leads, and every group boundary moves
        rolled = [torch.roll(a8d.view(torch.uint8), 128, 0).view(torch.float8_e4m3fn), torch.roll(sad, 128, 0).contiguous(),
                  torch.roll(idxd, 128, 0).contiguous()]
        got2 = out.cuda()
        yan.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((rolled[0], rolled[1]), (b8d, sbd), got2, rolled[2])
        assert torch.equal(torch.roll(got2, -128, 0), got)
    # the first group's rows through the plain entry point
    r0 = (group_rows[0] + 127) // 128 * 128
    plain = torch.zeros(r0, n, dtype=torch.bfloat16, device='cuda')
    yan.gemm_fp8_fp8_bf16_nt((a8d[:r0], sad[:r0].contiguous()), (b8d[0], sbd[0]), plain)
    assert float(yan.calc_diff(plain.float(), got[:r0].float())) < 1e-9


@pytest.mark.parametrize('rows,n,k,pad_blocks', testing.GROUPED_ROWS_ON_DEVICE_CASES)
def test_grouped_contiguous_kernel_that_picks_its_tile_height_on_the_device(rows, n, k, pad_blocks):
    """fp8_gemm_contiguous_rows_kernel on problems small enough for the oracle in full: with every group boundary on a
    multiple of 256 rows it runs 256 x 256 tiles, otherwise 128 x 256 ones; either way the oracle's result, the bits of the
    entry (which gives problems this small to other tiles: all tiles form the same sums), padding blocks untouched, and
    the same again under a compute-unit cap, where workgroups walk several tiles."""
    _announce('grouped rows on device', rows, n, k)
    (a8, sa), (b8, sb), out, idx = testing.make_grouped_contiguous_case(rows, n, k, seed=21, padding_blocks=pad_blocks)
    m, groups = a8.size(0), sum(1 for r in rows if r > 0)
    blocks = idx.view(-1, 128)[:, 0]
    halves = blocks[:len(blocks) // 2 * 2].view(-1, 2)
    two_group_rows = int(((halves[:, 0] != halves[:, 1]) & (halves >= 0).all(1)).sum())
    assert (two_group_rows == 0) == (rows == (512,) * 6)              # the first case is the one that runs 256-row tiles
    name, keys, arg_defs, code_template = testing.grouped_rows_on_device_plan(groups, n, k)
    from yan_amd.jit_kernels import m_grouped_gemm
    kernel = jit.build(name, arg_defs, jit.generate(m_grouped_gemm.includes, arg_defs, jit.cpp_format(code_template, keys)))
    a8d, sad, b8d, sbd, idxd = a8.cuda(), sa.cuda(), b8.cuda(), sb.cuda(), idx.cuda()
    ref = torch.from_numpy(oracle.m_grouped_gemm_contiguous_ref(_np_codes(a8), sa.numpy(), _np_codes(b8), sb.numpy(), idx.numpy(),
                                                                out_init=out.float().numpy()))
    via_entry = out.cuda()
    yan.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((a8d, sad), (b8d, sbd), via_entry, idxd)
    for cap in (yan.get_num_sms(), 8):
        got = out.cuda()
        assert kernel(a8d, sad, b8d, sbd, got, idxd, m, torch.cuda.current_stream(), cap, 0, sad.stride(0), sad.stride(1), 0, 0) == 0
        torch.cuda.synchronize()
        assert float(yan.calc_diff(got.float().cpu(), ref)) < 1e-3
        real = idx >= 0
        assert torch.equal(got.cpu()[~real], out[~real])
        assert bool(((got.float().cpu() - ref).abs() <= ref.abs() * 2.0 ** -7 + 1e-4 * ref.abs().max())[real].all())
        assert torch.equal(got, via_entry)


@pytest.mark.parametrize('groups,m_max,n,k,masked,expected_m', testing.GROUPED_MASKED_TEST_CASES)
def test_grouped_masked_parity(groups, m_max, n, k, masked, expected_m):
    """Masked layout against the oracle; rows at and beyond masked_m keep the caller's values; library == JIT."""
    (a8, sa), (b8, sb), out, mm = testing.make_grouped_masked_case(groups, m_max, n, k, masked, seed=6)
    a8d, sad, b8d, sbd, mmd = a8.cuda(), sa.cuda(), b8.cuda(), sb.cuda(), mm.cuda()
    got = out.cuda()
    assert yan.m_grouped_gemm_fp8_fp8_bf16_nt_masked((a8d, sad), (b8d, sbd), got, mmd, expected_m) is None
    if groups * m_max * n * k <= 2e10:
        ref = torch.from_numpy(oracle.m_grouped_gemm_masked_ref(_np_codes(a8), sa.numpy(), _np_codes(b8), sb.numpy(), mm.numpy(),
                                                                out_init=out.float().numpy()))
    else:
        ref = out.float()
        for g in range(groups):
            r = masked[g]
            ref[g, :r] = (testing.dequant_lhs(a8d[g, :r], sad[g, :r]) @ testing.dequant_rhs(b8d[g], sbd[g]).t()).cpu()
        g, r = 1, min(masked[1], 16)
        want = oracle.gemm_fp8_block_scaled_ref(_np_codes(a8[g, :r]), sa[g, :r].numpy(), _np_codes(b8[g]), sb[g].numpy())
        assert oracle.calc_diff(got[g, :r].float().cpu().numpy(), want) < 1e-3
    assert float(yan.calc_diff(got.float().cpu(), ref)) < 1e-3
    for g in range(groups):
        assert torch.equal(got[g, masked[g]:].cpu(), out[g, masked[g]:])  # masked-out rows untouched
        r = masked[g]
        if r:
            refg = ref[g, :r]
            assert bool(((got[g, :r].float().cpu() - refg).abs() <= refg.abs() * 2.0 ** -7 + 1e-4 * refg.abs().max()).all())
    via_lib = out.cuda()
    assert capi.m_grouped_gemm_fp8_fp8_bf16_nt_masked((a8d, sad), (b8d, sbd), via_lib, mmd, expected_m) == 0
    assert torch.equal(via_lib, got)


@pytest.mark.parametrize('m,n,k', [(1024, 1024, 1024), (255, 132, 72), (33, 4, 200), (257, 1028, 1096)])
def test_capi_dense_matches_oracle_and_jit(m, n, k):
    from yan_amd import capi
    _announce('capi dense', m, n, k)
    for dtype, fn, jit_fn in ((torch.bfloat16, capi.gemm_bf16_tn, yan.gemm_bf16_tn), (torch.half, capi.gemm_fp16_tn, yan.gemm_fp16_tn)):
        a, b, c = testing.make_bf16_case(m, n, k, seed=9, dtype=dtype, device='cuda')
        assert fn(a, b, c) == 0
        assert oracle.calc_diff(_np(c), oracle.gemm_bf16_tn_ref(_np(a), _np(b))) < BF16_TOL
        c2 = torch.zeros_like(c)
        jit_fn(a, b, c2)
        assert torch.equal(c, c2)            # same kernel source, same tile choice: same bits


@pytest.mark.parametrize('m,n,k', [(64, 256, 384), (129, 320, 128), (300, 96, 640), (257, 2112, 1024), (64, 4096, 7168), (1, 4096, 7168),
                                   (17, 4096, 1024), (33, 2112, 640)])
def test_capi_fp8_matches_oracle_and_jit(m, n, k):
    from yan_amd import capi
    _announce('capi fp8', m, n, k)
    (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=9, device='cuda')
    assert capi.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out) == 0
    assert oracle.calc_diff(_np(out), _fp8_ref(a8, sa, b8, sb)) < 1e-5
    out_cm = torch.zeros_like(out)
    assert capi.gemm_fp8_fp8_bf16_nt((a8, yan.get_col_major_tensor(sa)), (b8, sb), out_cm) == 0
    out_jit = torch.zeros_like(out)
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out_jit)
    assert torch.equal(out, out_cm)
    if yan.gemm.fp8_split_k_plan(m, n, k, yan.get_num_sms()) is None:
        assert torch.equal(out, out_jit)
    else:       # the JIT entry splits K; so does the library when it is handed a workspace: same plan, same bits
        out_split = torch.zeros_like(out)
        assert capi.gemm_fp8_fp8_bf16_nt_split_k((a8, sa), (b8, sb), out_split, capi.split_k_workspace()) == 0
        assert torch.equal(out_split, out_jit) and oracle.calc_diff(_np(out_jit), _fp8_ref(a8, sa, b8, sb)) < 1e-5


def test_entry_points_replay_correctly_from_a_captured_graph():
    """No entry point allocates, synchronises or keeps state, so a chain of them (quantiser -> FP8 GEMM, bf16 GEMM,
    fp32 GEMM with beta, masked grouped GEMM) can be captured once and replayed; every replay, with new contents in the
    static input buffers and eager work in between, must give the bits of an eager run on the same inputs."""
    _announce('graph replay')
    m, n, k = 256, 512, 512
    g = torch.Generator(device='cuda').manual_seed(77)
    x = torch.randn(m, k, device='cuda', generator=g).bfloat16()
    w = torch.randn(n, k, device='cuda', generator=g).bfloat16()
    w8, sw = yan.per_block_cast_to_fp8(w)
    xf_buf, wf_buf = torch.randn(k, m, device='cuda', generator=g), torch.randn(k, n, device='cuda', generator=g)
    (ga8, gsa), (gb8, gsb), _, masked = testing.make_grouped_masked_case(2, 128, n, k, (128, 40), seed=3, device='cuda')
    outs = {'fp8': torch.zeros(m, n, dtype=torch.bfloat16, device='cuda'), 'bf16': torch.zeros(m, n, dtype=torch.bfloat16, device='cuda'),
            'fp32': torch.zeros(m, n, device='cuda'), 'masked': torch.zeros(2, 128, n, dtype=torch.bfloat16, device='cuda')}

    def chain():
        a8, sa = yan.per_token_cast_to_fp8(x, col_major_scales=True)
        yan.gemm_fp8_fp8_bf16_nt((a8, sa), (w8, sw), outs['fp8'])
        yan.gemm_bf16_tn(x, w, outs['bf16'])
        yan.gemm_float_nt(xf_buf.t(), wf_buf.t(), outs['fp32'], alpha=0.5, beta=0.25)
        yan.m_grouped_gemm_fp8_fp8_bf16_nt_masked((ga8, gsa), (gb8, gsb), outs['masked'], masked, 128)

    def reset():
        for name, t in outs.items():
            t.fill_(1.0 if name == 'fp32' else 0.0)        # the fp32 GEMM reads c (beta != 0)

    reset()
    chain()                                                # loads every kernel before anything is captured
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        chain()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        chain()
    for rep in range(3):
        x.copy_(torch.randn(m, k, device='cuda', generator=g).bfloat16())
        xf_buf.copy_(torch.randn(k, m, device='cuda', generator=g))
        reset()
        graph.replay()
        torch.cuda.synchronize()
        replayed = {name: t.clone() for name, t in outs.items()}
        reset()
        chain()
        torch.cuda.synchronize()
        for name, t in outs.items():
            assert torch.equal(replayed[name], t), (rep, name)
        assert float(replayed['fp8'].float().abs().sum()) > 0 and float(replayed['masked'][1, 40:].float().abs().sum()) == 0


def test_split_k_replays_correctly_from_a_captured_graph():
    """Split-K launches captured into a graph: the workspace of the capture stream is made during the capture (a torch
    allocation and a fill kernel, both legal there) and every replay, with new inputs and eager split-K work on the other
    stream's workspace in between, gives the bits of an eager run."""
    _announce('split-k graph replay')
    (a8, sa), (b8, sb), out8 = testing.make_fp8_case(33, 2112, 5376, seed=8, device='cuda', gen_device='cuda')
    a, b, c = testing.make_bf16_case(100, 196, 3080, seed=9, scale=0.02, device='cuda', gen_device='cuda')
    assert yan.gemm.fp8_split_k_plan(33, 2112, 5376, yan.get_num_sms(), False) is not None

    def chain():
        yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out8)
        yan.gemm_bf16_tn(a, b, c)

    chain()                                                # loads the kernels
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        chain()
    g = torch.Generator(device='cuda').manual_seed(5)
    for rep in range(3):
        a.copy_((torch.randn(a.shape, device='cuda', generator=g) * 0.02).bfloat16())
        a8.copy_(torch.randn(a8.shape, device='cuda', generator=g).to(torch.float8_e4m3fn))
        out8.zero_()
        c.zero_()
        graph.replay()
        torch.cuda.synchronize()
        replayed = (out8.clone(), c.clone())
        out8.zero_()
        c.zero_()
        chain()
        torch.cuda.synchronize()
        assert torch.equal(replayed[0], out8) and torch.equal(replayed[1], c), rep
        assert float(out8.float().abs().sum()) > 0 and float(c.float().abs().sum()) > 0


def test_two_graphs_with_split_k_launches_do_not_share_a_workspace():
    """Two graphs captured one after the other, each with split-K launches: every capture gets a workspace of its own,
    zeroed by a node of its own graph, so the second graph replays correctly before the first has ever run, the two may be
    replayed on different streams at the same time, and eager launches in between use yet another workspace."""
    from yan_amd.jit_kernels import split_k
    _announce('two split-k graphs')
    (a8, sa), (b8, sb), out_1 = testing.make_fp8_case(33, 2112, 5376, seed=18, device='cuda', gen_device='cuda')
    (c8, sc), (d8, sd), out_2 = testing.make_fp8_case(64, 4096, 7168, seed=19, device='cuda', gen_device='cuda')
    assert yan.gemm.fp8_split_k_plan(33, 2112, 5376, yan.get_num_sms(), False) is not None
    assert yan.gemm.fp8_split_k_plan(64, 4096, 7168, yan.get_num_sms(), False) is not None
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out_1)
    yan.gemm_fp8_fp8_bf16_nt((c8, sc), (d8, sd), out_2)
    torch.cuda.synchronize()
    want_1, want_2 = out_1.clone(), out_2.clone()
    captures_before = len(split_k._book.captures)
    graph_1, graph_2 = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph_1):
        yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out_1)
        yan.gemm_fp8_fp8_bf16_nt((c8, sc), (d8, sd), out_2)
    with torch.cuda.graph(graph_2):
        yan.gemm_fp8_fp8_bf16_nt((c8, sc), (d8, sd), out_2)
        yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out_1)
    assert len(split_k._book.captures) == captures_before + 2
    ws = list(split_k._book.captures.values())[-2:]
    assert ws[0].data_ptr() != ws[1].data_ptr()
    assert all(w.data_ptr() != e.data_ptr() for w in ws for e in split_k._book.eager.values())
    for first, second in ((graph_2, graph_1), (graph_1, graph_2), (graph_2, graph_2)):
        for graph in (first, second):
            out_1.zero_()
            out_2.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out_1, want_1) and torch.equal(out_2, want_2)
            yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out_1)            # eager, on the stream's own workspace
    # a graph heals itself: counters left dirty by whatever ran before are zeroed by the graph's own first node
    ws[1][:split_k.SPLIT_K_COUNTER_BYTES].fill_(3)
    out_1.zero_()
    out_2.zero_()
    graph_2.replay()
    torch.cuda.synchronize()
    assert torch.equal(out_1, want_1) and torch.equal(out_2, want_2)


def test_a_workspace_whose_launch_failed_is_cleared_before_its_next_use(monkeypatch):
    """The entry points clear the arrival counters of a workspace after a launch on it reported an error: counters that
    are not zero would make the next launch store tiles early or never. With split-K switched off (YAN_SPLIT_K=0) the
    entry keeps no state and gives the bits of the unsplit kernel."""
    from yan_amd.jit_kernels import split_k
    _announce('suspect split-k workspace')
    (a8, sa), (b8, sb), out = testing.make_fp8_case(64, 4096, 7168, seed=20, device='cuda', gen_device='cuda')
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
    torch.cuda.synchronize()
    want = out.clone()
    workspace, token = split_k.split_k_workspace(out.device, yan.jit_kernels.utils.current_raw_stream())
    assert int(workspace[:split_k.SPLIT_K_COUNTER_BYTES].max()) == 0           # zero after a launch that ran to its end
    workspace[:split_k.SPLIT_K_COUNTER_BYTES].fill_(1)
    split_k.split_k_launch_failed(token)
    out.zero_()
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    assert int(workspace[:split_k.SPLIT_K_COUNTER_BYTES].max()) == 0
    monkeypatch.setenv('YAN_SPLIT_K', '0')
    eager_before = dict(split_k._book.eager)
    unsplit = torch.zeros_like(out)
    yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), unsplit)
    torch.cuda.synchronize()
    assert split_k._book.eager == eager_before
    ref = testing.dequant_lhs(a8, sa) @ testing.dequant_rhs(b8, sb).t()
    assert float(yan.calc_diff(unsplit.float(), ref)) < 1e-5 and float(yan.calc_diff(unsplit.float(), want.float())) < 1e-8


@pytest.mark.parametrize('m,n,k', testing.CAST_CHAIN_SHAPES)
def test_bf16_activation_entry_gives_the_bits_of_quantiser_then_gemm(m, n, k):
    """gemm_bf16_fp8_bf16_nt: one call, one `launch` that enqueues the quantiser and the GEMM, the codes in the entry's own
    scratch: the bits of per_token_cast_to_fp8 followed by gemm_fp8_fp8_bf16_nt, within the FP8 bar of the oracle's
    quantise-then-multiply on the same bf16 inputs, rows past m untouched, and nothing allocated per call."""
    from yan_amd.jit_kernels import gemm as fp8_entry
    _announce('bf16 activations', m, n, k)
    g = torch.Generator().manual_seed(97 + m)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = torch.randn(n, k, generator=g).bfloat16()
    b8, sb = testing.per_block_cast_to_fp8(w.float())
    xd, b8d, sbd = x.cuda(), b8.cuda(), sb.cuda()
    chained = fp8_entry.fp8_cast_chain_plan(m, n, k, yan.get_num_sms()) is not None
    assert chained == ((m, n, k) != (1100, 512, 4096))
    two = torch.zeros(m, n, dtype=torch.bfloat16, device='cuda')
    yan.gemm_fp8_fp8_bf16_nt(yan.per_token_cast_to_fp8(xd, col_major_scales=True), (b8d, sbd), two)
    one = torch.full((m + 3, n), 7.0, dtype=torch.bfloat16, device='cuda')
    yan.gemm_bf16_fp8_bf16_nt(xd, (b8d, sbd), one[:m])
    torch.cuda.synchronize()
    assert torch.equal(one[:m], two) and bool((one[m:] == 7.0).all())
    a8, sa = oracle.per_token_cast_to_fp8(x.float().numpy())
    ref = oracle.gemm_fp8_block_scaled_ref(a8, sa, _np(b8), _np(sb))
    assert oracle.calc_diff(_np(one[:m]), ref) < FP8_TOL
    if chained:
        target = one[:m]
        yan.gemm_bf16_fp8_bf16_nt(xd, (b8d, sbd), target)
        torch.cuda.synchronize()
        allocated = torch.cuda.memory_allocated()
        for _ in range(3):
            yan.gemm_bf16_fp8_bf16_nt(xd, (b8d, sbd), target)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == allocated and torch.equal(target, two)


def test_capi_seeded_random_shapes_against_device_references():
    """Breadth: 240 seeded random shapes through the C entries (every tile variant, ragged edges, k tails, leading
    dimensions), each against an fp32 / fp64 product of the same operands on the device. The oracle-based tests above
    pin the arithmetic; this one looks for a shape that breaks the tiling."""
    import random
    rng = random.Random(1234)
    _announce('capi random shapes')

    def rel_diff(x, y):
        x, y = x.double(), y.double()
        return float(1 - 2 * (x * y).sum() / ((x * x + y * y).sum() + 1e-300))

    for it in range(90):
        m = rng.choice([1, 7, 64, 255, 256, 257, 1000, 2048, 3000, 4100, 6000])
        n, k = 4 * rng.randint(1, 1500), 8 * rng.randint(1, 300)
        dtype = rng.choice([torch.bfloat16, torch.half])
        a, b = torch.randn(m, k, device='cuda').to(dtype), torch.randn(n, k, device='cuda').to(dtype)
        c = torch.full((m, n), 7.0, device='cuda', dtype=dtype)
        assert (capi.gemm_bf16_tn if dtype == torch.bfloat16 else capi.gemm_fp16_tn)(a, b, c) == 0
        assert rel_diff(c.float(), a.float() @ b.float().t()) < BF16_TOL, ('dense', m, n, k, dtype)
    for it in range(90):
        m = rng.choice([1, 5, 16, 17, 64, 100, 256, 300, 1024, 2050, 4096, 6000])
        n, k = 4 * rng.randint(1, 1800), 128 * rng.randint(1, 24)
        (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=it, device='cuda', gen_device='cuda')
        out.fill_(7.0)
        if rng.random() < 0.5:
            sa = yan.get_col_major_tensor(sa)
        assert capi.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out) == 0
        ref = testing.dequant_lhs(a8, sa) @ testing.dequant_rhs(b8, sb).t()
        assert rel_diff(out.float(), ref) < 1e-5, ('fp8', m, n, k)
    lib = capi.load()
    for it in range(60):
        m, n, k = 4 * rng.randint(1, 600), 4 * rng.randint(1, 600), rng.randint(0, 700)
        lda, ldb, ldc = m + 4 * rng.randint(0, 3), n + 4 * rng.randint(0, 3), n + 4 * rng.randint(0, 3)
        a_buf, b_buf = torch.randn(max(k, 1), lda, device='cuda'), torch.randn(max(k, 1), ldb, device='cuda')
        c_buf = torch.randn(m, ldc, device='cuda')
        alpha, beta = rng.choice([(1.0, 0.0), (0.5, 2.0), (-1.0, 1.0)])
        want = alpha * (a_buf[:k, :m].double().t() @ b_buf[:k, :n].double()) + (beta * c_buf[:, :n].double() if beta else 0)
        keep = c_buf[:, n:].clone()
        assert lib.yan_gemm_float_nt(m, n, k, alpha, a_buf.data_ptr(), lda, b_buf.data_ptr(), ldb, beta, c_buf.data_ptr(), ldc, None) == 0
        torch.cuda.synchronize()
        assert float((c_buf[:, :n].double() - want).abs().max()) < 1e-3, ('fp32', m, n, k, lda, ldb, ldc, alpha, beta)
        assert torch.equal(keep, c_buf[:, n:])


@pytest.mark.parametrize('cap', [0, 5])
def test_capi_fp8_beyond_the_memory_side_cache_ragged_and_capped(cap):
    """343 MB of FP8 operands with ragged edges through the C library: the persistent walk in region order (run-time N and
    K), uncapped and with 5 workgroups crossing the XCDs' ranges; every 512-row block against the dequantised product on
    the device."""
    m, n, k = 6690, 19292, 13824
    _announce('capi fp8 beyond the cache', m, n, k, cap)
    (a8, sa), (b8, sb), out = testing.make_fp8_case(m, n, k, seed=31, device='cuda', gen_device='cuda', col_major_scales=True)
    out.fill_(float('nan'))
    assert capi.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out, cap) == 0
    bt = testing.dequant_rhs(b8, sb).t().contiguous()
    for r0 in range(0, m, 512):
        ref = (testing.dequant_lhs(a8[r0:r0 + 512], sa[r0:r0 + 512]) @ bt).double()
        got = out[r0:r0 + 512].double()
        diff = 1 - 2 * (got * ref).sum().item() / ((got * got).sum().item() + (ref * ref).sum().item())
        assert diff < 1e-5, (r0, diff)


def test_capi_rejects_bad_sizes_on_device():
    from yan_amd import capi
    a = torch.zeros(64, 64, dtype=torch.bfloat16, device='cuda')
    lib = capi.load()
    null = None
    assert lib.yan_gemm_bf16_tn(64, 62, 64, a.data_ptr(), a.data_ptr(), a.data_ptr(), null) != 0
    assert lib.yan_gemm_bf16_tn(64, 64, 64, a.data_ptr(), a.data_ptr(), a.data_ptr(), null) == 0
    torch.cuda.synchronize()
