"""Writes tests/golden/gemm_small.npz (small seeded inputs and expected outputs for both GEMMs),
tests/golden/grouped_cast_small.npz (the grouped FP8 GEMM layouts and the two quantisers) and
tests/golden/float_small.npz (the fp32 GEMM with alpha / beta on raw buffers with leading dimensions).

The reference cannot produce these (no FP8 entry point, CUDA-only kernels, no fixtures of its own), so the
expected values come from the closed forms in oracle/gemm_oracle.py evaluated in fp64, cross-checked here against
the C triple loop before anything is written. Run from the repository root: `python tests/golden/make_golden.py`.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle                     # noqa: E402
from oracle import c_oracle       # noqa: E402


def main():
    rng = np.random.default_rng(20240607)
    out = {}
    # FP8 block-scaled, 64 x 256 x 384 (3 K blocks, 2 weight-scale rows), N(0,1) sources
    x = rng.standard_normal((64, 384)).astype(np.float32)
    w = rng.standard_normal((256, 384)).astype(np.float32)
    qa, sa = oracle.per_token_cast_to_fp8(x)
    qb, sb = oracle.per_block_cast_to_fp8(w)
    exp = oracle.gemm_fp8_block_scaled_ref(qa, sa, qb, sb, np.float64)
    assert oracle.calc_diff(c_oracle.gemm_fp8_nt(qa, sa, qb, sb), exp) < 1e-14
    out.update(fp8_lhs=qa, fp8_lhs_scales=sa, fp8_rhs=qb, fp8_rhs_scales=sb, fp8_expected_f64=exp)
    # bf16, 96 x 80 x 136 (k is not a multiple of 64: exercises the K tail)
    a = oracle.f32_to_bf16_bits(rng.standard_normal((96, 136)).astype(np.float32))
    b = oracle.f32_to_bf16_bits(rng.standard_normal((80, 136)).astype(np.float32))
    exp = oracle.gemm_bf16_tn_ref(oracle.bf16_bits_to_f32(a), oracle.bf16_bits_to_f32(b), np.float64)
    assert np.allclose(c_oracle.gemm_bf16_tn(a, b), exp, rtol=1e-12, atol=1e-12)
    out.update(bf16_a_bits=a, bf16_b_bits=b, bf16_expected_f64=exp)
    # exact-integer FP8 case with power-of-two scales, 40 x 192 x 256: a kernel must reproduce it bit for bit
    va = rng.integers(-4, 5, size=(40, 256)).astype(np.float32)
    vb = rng.integers(-4, 5, size=(192, 256)).astype(np.float32)
    isa = (2.0 ** rng.integers(-2, 3, size=(40, 2))).astype(np.float32)
    isb = (2.0 ** rng.integers(-2, 3, size=(2, 2))).astype(np.float32)
    ia, ib = oracle.e4m3fn_encode(va), oracle.e4m3fn_encode(vb)
    iexp = oracle.gemm_fp8_block_scaled_ref(ia, isa, ib, isb)
    assert np.array_equal(iexp, c_oracle.gemm_fp8_nt(ia, isa, ib, isb))
    out.update(int_lhs=ia, int_lhs_scales=isa, int_rhs=ib, int_rhs_scales=isb, int_expected=iexp)
    path = os.path.join(ROOT, 'tests', 'golden', 'gemm_small.npz')
    np.savez_compressed(path, **out)
    print('wrote', path, os.path.getsize(path), 'bytes')

    out = {}
    # quantisers: bf16 source, 130 x 256 (a ragged second block of rows for the per-block form), one all-zero group
    src = (rng.standard_normal((130, 256)) * 2.5).astype(np.float32)
    src[7, 128:] = 0
    bits = oracle.f32_to_bf16_bits(src)
    srcf = oracle.bf16_bits_to_f32(bits)
    tq, ts = oracle.per_token_cast_to_fp8(srcf)
    bq, bs = oracle.per_block_cast_to_fp8(srcf)
    out.update(cast_src_bf16_bits=bits, per_token_codes=tq, per_token_scales=ts, per_block_codes=bq, per_block_scales=bs)
    # grouped contiguous, exact integers with power-of-two scales: two groups of 128 rows and one block of padding
    # rows (index -1), n = 192, k = 256; masked: two groups of 40 rows, 40 and 7 of them valid
    G, n, k = 2, 192, 256
    wb = np.stack([oracle.e4m3fn_encode(rng.integers(-4, 5, size=(n, k)).astype(np.float32)) for _ in range(G)])
    wsb = (2.0 ** rng.integers(-2, 3, size=(G, 2, 2))).astype(np.float32)
    xa = oracle.e4m3fn_encode(rng.integers(-4, 5, size=(384, k)).astype(np.float32))
    xsa = (2.0 ** rng.integers(-2, 3, size=(384, 2))).astype(np.float32)
    idx = np.repeat(np.array([1, 0, -1], dtype=np.int32), 128)
    cexp = oracle.m_grouped_gemm_contiguous_ref(xa, xsa, wb, wsb, idx)
    for i in (0, 127, 128, 255):
        assert np.array_equal(cexp[i:i + 1], c_oracle.gemm_fp8_nt(xa[i:i + 1], xsa[i:i + 1], wb[idx[i]], wsb[idx[i]]))
    ma = np.stack([oracle.e4m3fn_encode(rng.integers(-4, 5, size=(40, k)).astype(np.float32)) for _ in range(G)])
    msa = (2.0 ** rng.integers(-2, 3, size=(G, 40, 2))).astype(np.float32)
    masked = np.array([40, 7], dtype=np.int32)
    mexp = oracle.m_grouped_gemm_masked_ref(ma, msa, wb, wsb, masked)
    assert np.array_equal(mexp[1, :7], c_oracle.gemm_fp8_nt(ma[1, :7], msa[1, :7], wb[1], wsb[1])) and not mexp[1, 7:].any()
    out.update(grouped_rhs=wb, grouped_rhs_scales=wsb, contiguous_lhs=xa, contiguous_lhs_scales=xsa, contiguous_m_indices=idx,
               contiguous_expected=cexp, masked_lhs=ma, masked_lhs_scales=msa, masked_m=masked, masked_expected=mexp)
    path = os.path.join(ROOT, 'tests', 'golden', 'grouped_cast_small.npz')
    np.savez_compressed(path, **out)
    print('wrote', path, os.path.getsize(path), 'bytes')


def float_fixture():
    """fp32 GEMM in the memory convention of the C ABI: A[i + t*lda], B[j + t*ldb], C[i*ldc + j]; 132 x 68 x 37 with
    padded leading dimensions, and an exact-integer 128 x 64 x 48 case."""
    rng = np.random.default_rng(20240921)
    m, n, k, lda, ldb, ldc = 132, 68, 37, 140, 72, 80
    a_buf = rng.standard_normal((k, lda)).astype(np.float32)
    b_buf = rng.standard_normal((k, ldb)).astype(np.float32)
    c_buf = rng.standard_normal((m, ldc)).astype(np.float32)
    alpha, beta = 0.75, -1.5
    exp = c_oracle.gemm_float_nt(m, n, k, alpha, a_buf, lda, b_buf, ldb, beta, c_buf, ldc).reshape(m, ldc)
    want = oracle.gemm_float_nt_ref(a_buf[:, :m].T, b_buf[:, :n].T, c_buf[:, :n], alpha, beta)
    assert np.allclose(exp[:, :n], want, rtol=1e-14, atol=1e-14)
    ia = rng.integers(-4, 5, size=(48, 128)).astype(np.float32)        # [k, m]: M contiguous
    ib = rng.integers(-4, 5, size=(48, 64)).astype(np.float32)
    ic = rng.integers(-8, 9, size=(128, 64)).astype(np.float32)
    iexp = oracle.gemm_float_nt_ref(ia.T, ib.T, ic, 0.5, 2.0)
    assert np.array_equal(iexp, iexp.astype(np.float32).astype(np.float64))       # exactly representable in fp32
    path = os.path.join(ROOT, 'tests', 'golden', 'float_small.npz')
    np.savez_compressed(path, dims=np.array([m, n, k, lda, ldb, ldc]), alpha_beta=np.array([alpha, beta]), a_buf=a_buf,
                        b_buf=b_buf, c_buf=c_buf, expected_f64=exp[:, :n], int_a=ia, int_b=ib, int_c=ic,
                        int_alpha_beta=np.array([0.5, 2.0]), int_expected=iexp)
    print('wrote', path, os.path.getsize(path), 'bytes')


if __name__ == '__main__':
    main()
    float_fixture()
