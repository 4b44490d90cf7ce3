"""Pins the CPU oracle (test infrastructure) before anything is compared against it.

The reference holds no golden vector for this path (its tests compare GPU results with GPU torch matmuls,
tests/test_cute.py:11-27), so every oracle function is pinned by what the mathematics fixes: closed forms,
exactly representable special cases, an independent C triple loop, torch's CPU casts as the library routine for
the number formats, and brute force on tiny inputs. Each check is chosen so that a plausible slip (wrong scale
index, transposed operand, dropped K block, wrong rounding mode) fails it.
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import c_oracle


# ----------------------------------------------------------------------------- calc_diff (yan/utils.py:109-113)
def test_calc_diff_invariants():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((17, 33))
    y = rng.standard_normal((17, 33))
    assert oracle.calc_diff(x, x) == 0.0
    assert oracle.calc_diff(x, -x) == 2.0
    assert oracle.calc_diff(x, np.zeros_like(x)) == 1.0
    assert oracle.calc_diff(x, y) == pytest.approx(oracle.calc_diff(y, x), abs=1e-15)
    # unlike a cosine it notices a pure scale error: 1 - 2s/(1+s^2)
    assert oracle.calc_diff(x, 2 * x) == pytest.approx(1 - 4 / 5, abs=1e-12)
    # hand-computed: x=(1,2), y=(2,1): 1 - 2*4/10
    assert oracle.calc_diff([1, 2], [2, 1]) == pytest.approx(0.2, abs=1e-15)


def test_calc_diff_matches_package():
    import yan_amd
    rng = np.random.default_rng(1)
    x, y = rng.standard_normal(1000), rng.standard_normal(1000)
    got = float(yan_amd.calc_diff(torch.from_numpy(x), torch.from_numpy(y)))
    assert got == pytest.approx(oracle.calc_diff(x, y), abs=1e-14)


# ----------------------------------------------------------------------------- number formats
def test_e4m3_known_answers():
    t = oracle.e4m3fn_decode_table()
    assert t[0x00] == 0 and t[0x80] == 0 and np.signbit(t[0x80])
    assert t[0x7E] == 448.0 and t[0xFE] == -448.0
    assert np.isnan(t[0x7F]) and np.isnan(t[0xFF])
    assert t[0x08] == 2.0 ** -6          # smallest normal
    assert t[0x01] == 2.0 ** -9          # smallest subnormal
    assert t[0x07] == 7 * 2.0 ** -9      # largest subnormal
    assert t[0x38] == 1.0 and t[0x40] == 2.0 and t[0x44] == 3.0 and t[0x30] == 0.5
    assert np.isfinite(t).sum() == 254


def test_e4m3_table_matches_torch_cpu_cast():
    ours = oracle.e4m3fn_decode_table()
    lib = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(ours), np.isnan(lib))
    assert np.array_equal(ours[~np.isnan(ours)], lib[~np.isnan(lib)])


def test_e4m3_encode_matches_torch_cpu_cast():
    rng = np.random.default_rng(2)
    x = np.concatenate([(rng.standard_normal(50000) * s).astype(np.float32) for s in (1e-3, 1e-2, 1, 30, 300)])
    special = np.array([0, -0.0, 448, 449, 463.9, 464, 464.0001, 465, 480, 1e9, -464, -465, np.inf, -np.inf, np.nan,
                        2 ** -9, 2 ** -10, 1.5 * 2 ** -10, 0.99 * 2 ** -10, 17, 18, 19, 20, 22, 26, 30], dtype=np.float32)
    x = np.concatenate([x, special])
    lib = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(oracle.e4m3fn_encode(x), lib)
    # every finite code survives a decode -> encode round trip
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    assert np.array_equal(oracle.e4m3fn_encode(oracle.e4m3fn_decode(codes)), codes)
    # ties go to even: 17 lies between 16 (0x58) and 18 (0x59)
    assert oracle.e4m3fn_encode(np.float32(17))[()] == 0x58 and oracle.e4m3fn_encode(np.float32(19))[()] == 0x5A


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(100000).astype(np.float32) * 100,
                        np.array([1.0, 1.00390625, 1.01171875, 3.0e38, -1e-30, 0.0], dtype=np.float32)])
    lib = torch.from_numpy(x).bfloat16().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16_bits(x), lib)
    assert np.array_equal(oracle.bf16_bits_to_f32(lib), torch.from_numpy(x).bfloat16().float().numpy())
    # 1 + 2^-8 is a tie between 1.0 and 1 + 2^-7: even mantissa wins
    assert oracle.bf16_round(np.float32(1.00390625))[()] == 1.0
    assert oracle.bf16_round(np.float32(1.01171875))[()] == np.float32(1.015625)


# ----------------------------------------------------------------------------- quantisers (harness recipes)
@pytest.mark.parametrize('dist', ['normal', 'outlier'])
def test_quantisers_bounds_and_roundtrip(dist):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((40, 384)).astype(np.float32)
    w = rng.standard_normal((200, 384)).astype(np.float32)
    if dist == 'outlier':
        x = (rng.random((40, 384)) * 8 - 4).astype(np.float32)
        x = np.where(rng.random(x.shape) < 0.01, x * 50, x).astype(np.float32)
    qa, sa = oracle.per_token_cast_to_fp8(x)
    qb, sb = oracle.per_block_cast_to_fp8(w)
    assert qa.shape == x.shape and sa.shape == (40, 3) and qb.shape == w.shape and sb.shape == (2, 3)
    for q in (qa, qb):
        d = oracle.e4m3fn_decode(q)
        assert np.isfinite(d).all() and np.abs(d).max() <= 448.0
    # every group reaches the top code, and the error per element is at most half an e4m3 step at 448: amax/448*16
    amax = np.abs(x).reshape(40, 3, 128).max(-1)
    assert np.allclose(sa * 448, amax, rtol=1e-6)
    err = np.abs(oracle.dequant_lhs(qa, sa) - x).reshape(40, 3, 128).max(-1)
    assert (err <= amax * 2.0 ** -4 * (1 + 1e-6)).all()
    errb = np.abs(oracle.dequant_rhs(qb, sb) - w)
    assert errb.max() <= np.abs(w).max() * 2.0 ** -4
    # tiny groups clamp to amax 1e-4 instead of dividing by zero
    qz, sz = oracle.per_token_cast_to_fp8(np.zeros((2, 128), np.float32))
    assert (qz == 0).all() and np.allclose(sz, 1e-4 / 448)


def test_quantisers_match_package_harness():
    import harness as testing
    g = torch.Generator().manual_seed(5)
    # bf16-valued sources: few mantissa bits, so x * factor lands exactly on rounding ties now and then
    x, w = torch.randn(48, 256, generator=g).bfloat16().float(), torch.randn(160, 256, generator=g).bfloat16().float()
    qa, sa = testing.per_token_cast_to_fp8(x)
    qb, sb = testing.per_block_cast_to_fp8(w)
    oa, osa = oracle.per_token_cast_to_fp8(x.numpy())
    ob, osb = oracle.per_block_cast_to_fp8(w.numpy())
    assert np.array_equal(qa.view(torch.uint8).numpy(), oa) and np.array_equal(sa.numpy(), osa)
    assert np.array_equal(qb.view(torch.uint8).numpy(), ob) and np.array_equal(sb.numpy(), osb)
    assert np.array_equal(testing.dequant_lhs(qa, sa).numpy(), oracle.dequant_lhs(oa, osa))
    assert np.array_equal(testing.dequant_rhs(qb, sb).numpy(), oracle.dequant_rhs(ob, osb))


# ----------------------------------------------------------------------------- bf16 GEMM
def _bf16(x):
    return oracle.bf16_round(np.asarray(x, np.float32))


def test_bf16_gemm_closed_forms():
    # the ones pattern of the reference's commented smoke case (yan/jit_kernels/cute_gemm.py:74-79):
    # a[:, ::4] = 1, b[:, ::3] = 1  =>  c = #multiples of 12 below k = ceil(k / 12)
    m, n, k = 128, 256, 256
    a, b = np.zeros((m, k), np.float32), np.zeros((n, k), np.float32)
    a[:, ::4] = 1
    b[:, ::3] = 1
    assert np.array_equal(oracle.gemm_bf16_tn_ref(a, b), np.full((m, n), -(-k // 12), np.float32))
    # identity on the B side returns A; a transposed-operand slip would return A.T-shaped garbage or fail
    rng = np.random.default_rng(6)
    a = _bf16(rng.standard_normal((7, 16)))
    assert np.array_equal(oracle.gemm_bf16_tn_ref(a, np.eye(16, dtype=np.float32)), a)
    # one-hot rows pick single products: c[i, j] = a[i, p] * b[j, p]
    b = np.zeros((5, 16), np.float32)
    b[np.arange(5), [3, 1, 4, 1, 5]] = [2, -1, 0.5, 4, 8]
    want = a[:, [3, 1, 4, 1, 5]] * np.array([2, -1, 0.5, 4, 8], np.float32)
    assert np.array_equal(oracle.gemm_bf16_tn_ref(a, b), want)


def test_bf16_gemm_numpy_vs_c_triple_loop_vs_bruteforce():
    rng = np.random.default_rng(7)
    a, b = _bf16(rng.standard_normal((33, 72))), _bf16(rng.standard_normal((20, 72)))
    c64 = c_oracle.gemm_bf16_tn(oracle.f32_to_bf16_bits(a), oracle.f32_to_bf16_bits(b))
    brute = np.array([[sum(float(a[i, t]) * float(b[j, t]) for t in range(72)) for j in range(20)] for i in range(33)])
    assert np.allclose(c64, brute, rtol=1e-13, atol=1e-13)
    assert oracle.calc_diff(oracle.gemm_bf16_tn_ref(a, b), c64) < 1e-12
    assert np.allclose(oracle.gemm_bf16_tn_ref(a, b, np.float64), c64, rtol=1e-12, atol=1e-12)
    # K-split additivity and linearity in A
    full = oracle.gemm_bf16_tn_ref(a, b, np.float64)
    assert np.allclose(full, oracle.gemm_bf16_tn_ref(a[:, :40], b[:, :40], np.float64)
                       + oracle.gemm_bf16_tn_ref(a[:, 40:], b[:, 40:], np.float64))
    assert np.allclose(oracle.gemm_bf16_tn_ref(2 * a, b, np.float64), 2 * full)


# ----------------------------------------------------------------------------- fp32 GEMM with alpha / beta
def test_float_gemm_closed_forms_and_memory_convention():
    rng = np.random.default_rng(21)
    # the ones pattern again: exact small integers, so alpha and beta show up exactly
    m, n, k = 8, 12, 48
    a, b = np.zeros((m, k), np.float32), np.zeros((n, k), np.float32)
    a[:, ::4] = 1
    b[:, ::3] = 1
    c = np.arange(m * n, dtype=np.float32).reshape(m, n)
    assert np.array_equal(oracle.gemm_float_nt_ref(a, b), np.full((m, n), 4.0))
    assert np.array_equal(oracle.gemm_float_nt_ref(a, b, c, alpha=0.5, beta=-2.0), 2.0 - 2.0 * c)
    # beta == 0 ignores what c held (NaN included); identity on the B side returns alpha * A
    a = rng.standard_normal((7, 16)).astype(np.float32)
    assert np.array_equal(oracle.gemm_float_nt_ref(a, np.eye(16, dtype=np.float32), np.full((7, 16), np.nan), 3.0, 0.0), 3.0 * a.astype(np.float64))
    # raw-buffer triple loop in the C ABI's convention (A[i + t*lda], B[j + t*ldb], C[i*ldc + j]) against the
    # logical-array form: a swapped leading dimension or a transposed operand fails this
    m, n, k, lda, ldb, ldc = 8, 12, 5, 12, 16, 20
    a_buf = rng.standard_normal((k, lda)).astype(np.float32)
    b_buf = rng.standard_normal((k, ldb)).astype(np.float32)
    c_buf = rng.standard_normal((m, ldc)).astype(np.float32)
    for alpha, beta in ((1.0, 0.0), (0.5, 2.0), (-1.25, 1.0)):
        got = c_oracle.gemm_float_nt(m, n, k, alpha, a_buf, lda, b_buf, ldb, beta, c_buf, ldc).reshape(m, ldc)
        want = oracle.gemm_float_nt_ref(a_buf[:, :m].T, b_buf[:, :n].T, c_buf[:, :n], alpha, beta)
        assert np.allclose(got[:, :n], want, rtol=1e-14, atol=1e-14)
        assert not got[:, n:].any()                     # outside the m x n window nothing is written
        brute = np.array([[alpha * sum(float(a_buf[t, i]) * float(b_buf[t, j]) for t in range(k)) + (beta * float(c_buf[i, j]) if beta else 0.0)
                           for j in range(n)] for i in range(m)])
        assert np.allclose(want, brute, rtol=1e-13, atol=1e-13)
    # linearity in alpha and in beta, K-split additivity
    a, b, c = a_buf[:, :m].T, b_buf[:, :n].T, c_buf[:, :n]
    full = oracle.gemm_float_nt_ref(a, b, c, 1.0, 1.0)
    assert np.allclose(full, oracle.gemm_float_nt_ref(a[:, :2], b[:, :2]) + oracle.gemm_float_nt_ref(a[:, 2:], b[:, 2:], c, 1.0, 1.0))
    assert np.allclose(oracle.gemm_float_nt_ref(a, b, c, 2.0, 3.0), 2.0 * oracle.gemm_float_nt_ref(a, b) + 3.0 * c.astype(np.float64))


# ----------------------------------------------------------------------------- FP8 block-scaled GEMM
def _small_int_codes(rng, shape):
    """e4m3 codes of values in {-4..4}: every product and every 128-term sum is an exact small integer in fp32."""
    vals = rng.integers(-4, 5, size=shape).astype(np.float32)
    return oracle.e4m3fn_encode(vals), vals


def test_fp8_unit_scales_reduce_to_exact_integer_gemm():
    rng = np.random.default_rng(8)
    qa, va = _small_int_codes(rng, (24, 384))
    qb, vb = _small_int_codes(rng, (200, 384))
    sa, sb = np.ones((24, 3), np.float32), np.ones((2, 3), np.float32)
    want = (va.astype(np.int64) @ vb.astype(np.int64).T).astype(np.float64)
    assert np.array_equal(oracle.gemm_fp8_block_scaled_ref(qa, sa, qb, sb), want)
    assert np.array_equal(oracle.gemm_fp8_blockwise_f32(qa, sa, qb, sb), want)
    assert np.array_equal(c_oracle.gemm_fp8_nt(qa, sa, qb, sb), want)


def test_fp8_power_of_two_scales_are_exact_and_index_the_right_block():
    rng = np.random.default_rng(9)
    m, n, k = 16, 256, 512
    qa, va = _small_int_codes(rng, (m, k))
    qb, vb = _small_int_codes(rng, (n, k))
    sa = 2.0 ** rng.integers(-3, 4, size=(m, k // 128)).astype(np.float32)
    sb = 2.0 ** rng.integers(-3, 4, size=(n // 128, k // 128)).astype(np.float32)
    # closed form with explicit indices sA[i, kb], sB[j // 128, kb]
    want = np.zeros((m, n))
    for kb in range(k // 128):
        part = va[:, kb * 128:(kb + 1) * 128].astype(np.float64) @ vb[:, kb * 128:(kb + 1) * 128].astype(np.float64).T
        for jb in range(n // 128):
            want[:, jb * 128:(jb + 1) * 128] += part[:, jb * 128:(jb + 1) * 128] * sa[:, kb:kb + 1] * sb[jb, kb]
    for got in (oracle.gemm_fp8_block_scaled_ref(qa, sa, qb, sb), oracle.gemm_fp8_blockwise_f32(qa, sa, qb, sb),
                c_oracle.gemm_fp8_nt(qa, sa, qb, sb)):
        assert np.array_equal(got, want)
    # a transposed scale table (sB[kb, j//128]) or a row/column slip in sA must change the answer
    assert not np.array_equal(oracle.gemm_fp8_block_scaled_ref(qa, sa[::-1].copy(), qb, sb), want)


def test_fp8_single_k_block_isolates_scale_indexing():
    rng = np.random.default_rng(10)
    m, n, k = 8, 320, 640            # n is not a multiple of 128: the last scale row covers 64 rows
    qa, va = _small_int_codes(rng, (m, k))
    qb, vb = _small_int_codes(rng, (n, k))
    sa = rng.random((m, 5)).astype(np.float32) + 0.5
    sb = rng.random((3, 5)).astype(np.float32) + 0.5
    kb = 3
    qa0, qb0 = np.zeros_like(qa), qb.copy()
    qa0[:, kb * 128:(kb + 1) * 128] = qa[:, kb * 128:(kb + 1) * 128]
    part = va[:, kb * 128:(kb + 1) * 128].astype(np.float64) @ vb[:, kb * 128:(kb + 1) * 128].astype(np.float64).T
    want = part * sa[:, kb].astype(np.float64)[:, None] * np.repeat(sb[:, kb].astype(np.float64), 128)[:n][None, :]
    assert np.allclose(oracle.gemm_fp8_block_scaled_ref(qa0, sa, qb0, sb, np.float64), want, rtol=1e-6, atol=1e-4)    # dequantises in fp32
    assert np.allclose(c_oracle.gemm_fp8_nt(qa0, sa, qb0, sb), want, rtol=1e-12)
    assert np.allclose(oracle.gemm_fp8_blockwise_f32(qa0, sa, qb0, sb), want, rtol=1e-6, atol=1e-4)


def test_fp8_three_evaluations_agree_on_random_data_and_track_the_unquantised_product():
    rng = np.random.default_rng(11)
    x, w = rng.standard_normal((48, 512)).astype(np.float32), rng.standard_normal((192, 512)).astype(np.float32)
    qa, sa = oracle.per_token_cast_to_fp8(x)
    qb, sb = oracle.per_block_cast_to_fp8(w)
    d64 = oracle.gemm_fp8_block_scaled_ref(qa, sa, qb, sb, np.float64)
    assert oracle.calc_diff(c_oracle.gemm_fp8_nt(qa, sa, qb, sb), d64) < 1e-14
    assert oracle.calc_diff(oracle.gemm_fp8_block_scaled_ref(qa, sa, qb, sb), d64) < 1e-12
    assert oracle.calc_diff(oracle.gemm_fp8_blockwise_f32(qa, sa, qb, sb), d64) < 1e-12
    # quantisation noise of e4m3 at this depth, not a bug-sized difference
    assert 1e-5 < oracle.calc_diff(d64, x.astype(np.float64) @ w.astype(np.float64).T) < 2e-3
    # strided (token-contiguous) scales are the same numbers
    sa_cm = np.asfortranarray(sa)
    assert np.array_equal(c_oracle.gemm_fp8_nt(qa, sa_cm, qb, sb), c_oracle.gemm_fp8_nt(qa, sa, qb, sb))


# ----------------------------------------------------------------------------- committed fixtures
def test_grouped_forms_against_row_by_row_brute_force():
    """The grouped oracles are the plain one applied per group. Pinned by: the C triple loop on every row taken alone
    with the weight matrix its index names (small-integer data and power-of-two scales, so everything is exact);
    one group == the plain form; relabelling the groups together with their weights changes nothing; rows that are
    padding (negative index) or beyond masked_m keep what the caller had there."""
    rng = np.random.default_rng(21)
    G, n, k = 3, 136, 256
    qb = np.stack([_small_int_codes(rng, (n, k))[0] for _ in range(G)])
    sb = 2.0 ** rng.integers(-2, 3, size=(G, 2, k // 128)).astype(np.float32)
    m = 24
    qa, _ = _small_int_codes(rng, (m, k))
    sa = 2.0 ** rng.integers(-2, 3, size=(m, k // 128)).astype(np.float32)
    idx = np.array([0] * 8 + [2] * 8 + [-1] * 4 + [1] * 4, dtype=np.int32)
    init = rng.standard_normal((m, n)).astype(np.float32)
    got = oracle.m_grouped_gemm_contiguous_ref(qa, sa, qb, sb, idx, out_init=init)
    for i in range(m):
        if idx[i] < 0:
            assert np.array_equal(got[i], init[i])
        else:
            want = c_oracle.gemm_fp8_nt(qa[i:i + 1], sa[i:i + 1], qb[idx[i]], sb[idx[i]])
            assert np.array_equal(got[i:i + 1], want)
    # one group: the plain form
    one = oracle.m_grouped_gemm_contiguous_ref(qa, sa, qb[1:2], sb[1:2], np.zeros(m, np.int32))
    assert np.array_equal(one, oracle.gemm_fp8_block_scaled_ref(qa, sa, qb[1], sb[1]))
    # relabel groups 0 <-> 2 and swap their weights: same answer; swap only the labels: different answer
    perm = np.array([2, 1, 0])
    relabeled = np.where(idx >= 0, perm[np.maximum(idx, 0)], idx).astype(np.int32)
    assert np.array_equal(oracle.m_grouped_gemm_contiguous_ref(qa, sa, qb[perm], sb[perm], relabeled, out_init=init), got)
    assert not np.array_equal(oracle.m_grouped_gemm_contiguous_ref(qa, sa, qb, sb, relabeled, out_init=init), got)

    # masked layout
    m_max = 10
    qa3 = np.stack([_small_int_codes(rng, (m_max, k))[0] for _ in range(G)])
    sa3 = 2.0 ** rng.integers(-2, 3, size=(G, m_max, k // 128)).astype(np.float32)
    masked = np.array([10, 0, 3], dtype=np.int32)
    init3 = rng.standard_normal((G, m_max, n)).astype(np.float32)
    got3 = oracle.m_grouped_gemm_masked_ref(qa3, sa3, qb, sb, masked, out_init=init3)
    for g in range(G):
        for i in range(m_max):
            if i >= masked[g]:
                assert np.array_equal(got3[g, i], init3[g, i])
            else:
                assert np.array_equal(got3[g, i:i + 1], c_oracle.gemm_fp8_nt(qa3[g, i:i + 1], sa3[g, i:i + 1], qb[g], sb[g]))


def test_golden_fixtures_reproduce(repo_root):
    import os
    path = os.path.join(repo_root, 'tests', 'golden', 'gemm_small.npz')
    z = np.load(path)
    got = oracle.gemm_fp8_block_scaled_ref(z['fp8_lhs'], z['fp8_lhs_scales'], z['fp8_rhs'], z['fp8_rhs_scales'], np.float64)
    assert np.array_equal(got, z['fp8_expected_f64'])
    assert oracle.calc_diff(c_oracle.gemm_fp8_nt(z['fp8_lhs'], z['fp8_lhs_scales'], z['fp8_rhs'], z['fp8_rhs_scales']),
                            z['fp8_expected_f64']) < 1e-14
    a, b = oracle.bf16_bits_to_f32(z['bf16_a_bits']), oracle.bf16_bits_to_f32(z['bf16_b_bits'])
    assert np.array_equal(oracle.gemm_bf16_tn_ref(a, b, np.float64), z['bf16_expected_f64'])
    assert np.allclose(c_oracle.gemm_bf16_tn(z['bf16_a_bits'], z['bf16_b_bits']), z['bf16_expected_f64'], rtol=1e-12, atol=1e-12)
    assert np.array_equal(z['int_expected'], oracle.gemm_fp8_block_scaled_ref(z['int_lhs'], z['int_lhs_scales'], z['int_rhs'], z['int_rhs_scales']))


def test_float_fixture_reproduces(repo_root):
    import os
    z = np.load(os.path.join(repo_root, 'tests', 'golden', 'float_small.npz'))
    m, n, k, lda, ldb, ldc = (int(v) for v in z['dims'])
    alpha, beta = (float(v) for v in z['alpha_beta'])
    got = c_oracle.gemm_float_nt(m, n, k, alpha, z['a_buf'], lda, z['b_buf'], ldb, beta, z['c_buf'], ldc).reshape(m, ldc)
    assert np.array_equal(got[:, :n], z['expected_f64'])
    want = oracle.gemm_float_nt_ref(z['a_buf'][:, :m].T, z['b_buf'][:, :n].T, z['c_buf'][:, :n], alpha, beta)
    assert np.allclose(want, z['expected_f64'], rtol=1e-14, atol=1e-14)
    ia, ib = (float(v) for v in z['int_alpha_beta'])
    assert np.array_equal(oracle.gemm_float_nt_ref(z['int_a'].T, z['int_b'].T, z['int_c'], ia, ib), z['int_expected'])


def test_grouped_and_cast_fixtures_reproduce(repo_root):
    import os
    z = np.load(os.path.join(repo_root, 'tests', 'golden', 'grouped_cast_small.npz'))
    src = oracle.bf16_bits_to_f32(z['cast_src_bf16_bits'])
    tq, ts = oracle.per_token_cast_to_fp8(src)
    bq, bs = oracle.per_block_cast_to_fp8(src)
    assert np.array_equal(tq, z['per_token_codes']) and np.array_equal(ts, z['per_token_scales'])
    assert np.array_equal(bq, z['per_block_codes']) and np.array_equal(bs, z['per_block_scales'])
    # torch's op chain on the same source: `448.0 / amax` is evaluated there as reciprocal(amax) * 448, one ulp away
    # from the correctly rounded quotient for some amax, so a code moves where x * factor lands on a rounding boundary
    # (bf16-valued sources make exact ties common); the scales, a plain division, are identical
    xt = torch.from_numpy(src)
    amax = xt.view(130, 2, 128).abs().amax(dim=2).clamp(1e-4)
    q = (xt.view(130, 2, 128) * (448.0 / amax).unsqueeze(2)).to(torch.float8_e4m3fn).view(130, 256)
    moved = q.view(torch.uint8).numpy() != z['per_token_codes']
    assert moved.mean() < 2e-3 and np.array_equal((amax / 448.0).numpy(), z['per_token_scales'])
    exact = (xt.view(130, 2, 128) * (torch.tensor(448.0) / amax).unsqueeze(2)).to(torch.float8_e4m3fn).view(130, 256)
    assert np.array_equal(exact.view(torch.uint8).numpy(), z['per_token_codes'])      # with a true division: bit for bit
    assert np.array_equal(oracle.m_grouped_gemm_contiguous_ref(z['contiguous_lhs'], z['contiguous_lhs_scales'], z['grouped_rhs'],
                                                               z['grouped_rhs_scales'], z['contiguous_m_indices']), z['contiguous_expected'])
    assert np.array_equal(oracle.m_grouped_gemm_masked_ref(z['masked_lhs'], z['masked_lhs_scales'], z['grouped_rhs'],
                                                           z['grouped_rhs_scales'], z['masked_m']), z['masked_expected'])
