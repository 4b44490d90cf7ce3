"""numpy oracle for the bf16 GEMM and the FP8 e4m3 block-scaled GEMM. TEST INFRASTRUCTURE, never the product path.

What each function restates (paths relative to the reference tree):
  calc_diff                  yan/utils.py:109-113                      1 - 2<x,y>/(|x|^2+|y|^2) in fp64
  gemm_bf16_tn_ref           yan/jit_kernels/cute_gemm.py:21-38,84      c = a @ b.T; tests/test_cute.py:14 uses torch's matmul
                                                                       as the expected value, i.e. the textbook contraction
  gemm_fp8_block_scaled_ref  yan/jit_kernels/gemm.py:9-31 (operand names, BLOCK_K = 128),
                             yan/include/gemm/fp8_gemm.cuh:48-61        one A scale per row per 128-K, one B scale per
                                                                       128x128 block; the reference has no executable FP8
                                                                       path, so the closed form is the oracle
  gemm_float_nt_ref          yan/jit_kernels/simple_gemm.py:18-57, yan/include/gemm/simple_gemm.cuh:191 (axpby):
                             alpha * a @ b.T + beta * c on logical [m,k] / [n,k] / [m,n] arrays, in fp64
  m_grouped_gemm_contiguous_ref,
  m_grouped_gemm_masked_ref  yan/include/gemm/scheduler.cuh:7-11,31-48, yan/include/gemm/fp8_gemm.cuh:41 (the GemmType
                             enumerators and grouped_layout hook; the reference has no grouped entry point and no test):
                             gemm_fp8_block_scaled_ref applied per group, row by row -- the row's group picks the weight
                             matrix; rows with a negative index / beyond masked_m keep the caller's values
  e4m3fn_decode / encode     OCP FP8 E4M3 (the dtype named in yan/jit/template.py:18): 1-4-3, bias 7, no inf, S.1111.111 NaN
  per_token_cast_to_fp8,
  per_block_cast_to_fp8      harness-side quantisers of the benchmark configs (amax over 1x128 / 128x128 groups,
                             clamp 1e-4, x*448/amax -> e4m3fn, scale = amax/448); not part of the reference tree

Pinned by tests/test_oracle.py: closed forms (identity, ones pattern of cute_gemm.py:74-79, unit and power-of-two
scales giving exact integer results, single-K-block scale isolation), the independent C triple loop in
gemm_oracle.c, brute force on tiny inputs, the 256-entry e4m3 table against torch's CPU cast, and the committed
fixtures under tests/golden/. The reference holds no golden vectors for this path. The grouped forms are pinned
against a row-by-row brute force (every row multiplied with the weight matrix its index names, one row at a time),
against the plain form for a single group, and by permuting the groups. gemm_float_nt_ref is pinned by closed forms
(identity, the ones pattern, alpha / beta linearity) and, together with the memory convention of the C ABI, by the
raw-buffer triple loop oracle_gemm_float_nt in gemm_oracle.c.
"""
import numpy as np

__all__ = ['calc_diff', 'e4m3fn_decode_table', 'e4m3fn_decode', 'e4m3fn_encode', 'bf16_bits_to_f32', 'f32_to_bf16_bits',
           'bf16_round', 'per_token_cast_to_fp8', 'per_block_cast_to_fp8', 'dequant_lhs', 'dequant_rhs',
           'gemm_bf16_tn_ref', 'gemm_float_nt_ref', 'gemm_fp8_block_scaled_ref', 'gemm_fp8_blockwise_f32',
           'm_grouped_gemm_contiguous_ref', 'm_grouped_gemm_masked_ref']

FP8_MAX = 448.0


def calc_diff(x, y) -> float:
    x = np.asarray(x, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    return float(1.0 - 2.0 * (x * y).sum() / (x * x + y * y).sum())


# ----------------------------------------------------------------------------- number formats
def e4m3fn_decode_table() -> np.ndarray:
    """All 256 e4m3fn codes as fp32: sign(1) exp(4, bias 7) mant(3); exp 0 is subnormal; 0x7f / 0xff are NaN."""
    code = np.arange(256, dtype=np.int64)
    sign = np.where(code & 0x80, -1.0, 1.0)
    exp = (code >> 3) & 0xF
    man = (code & 0x7).astype(np.float64)
    val = np.where(exp == 0, man / 8.0 * 2.0 ** -6, (1.0 + man / 8.0) * 2.0 ** (exp - 7.0))
    val = sign * val
    val[(code & 0x7F) == 0x7F] = np.nan
    return val.astype(np.float32)


_E4M3_TABLE = e4m3fn_decode_table()


def e4m3fn_decode(codes) -> np.ndarray:
    return _E4M3_TABLE[np.asarray(codes, dtype=np.uint8)]


def e4m3fn_encode(x) -> np.ndarray:
    """fp32 -> e4m3fn code, round to nearest even; magnitudes that round above 448 become NaN (0x7f), which is how
    the unsaturated OCP conversion behaves. Works by nearest-neighbour search over the 127 finite magnitudes."""
    x = np.asarray(x, dtype=np.float32)
    mags = _E4M3_TABLE[:0x7F].astype(np.float64)          # 0 .. 448, strictly increasing
    ax = np.abs(x.astype(np.float64))
    hi = np.clip(np.searchsorted(mags, ax, side='left'), 1, 0x7E)
    lo = hi - 1
    d_lo, d_hi = ax - mags[lo], mags[hi] - ax
    pick_hi = (d_hi < d_lo) | ((d_hi == d_lo) & (hi % 2 == 0))     # tie -> even code (even mantissa)
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    # beyond the largest finite value: past the halfway point 464 to the (non-existent) next step 480 is NaN;
    # exactly 464 ties to the even mantissa, 448
    code = np.where(ax > 464.0, 0x7F, code).astype(np.uint8)
    code = np.where(np.isnan(x), 0x7F, code).astype(np.uint8)
    return (code | np.where(np.signbit(x), 0x80, 0).astype(np.uint8)).astype(np.uint8)


def bf16_bits_to_f32(bits) -> np.ndarray:
    return (np.asarray(bits).astype(np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(x) -> np.ndarray:
    """fp32 -> bf16 bit pattern, round to nearest even (finite inputs)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)


def bf16_round(x) -> np.ndarray:
    return bf16_bits_to_f32(f32_to_bf16_bits(x))


# ----------------------------------------------------------------------------- quantisers (harness)
def _grouped_amax(x, gm, gk):
    m, k = x.shape
    return np.abs(x).reshape(m // gm, gm, k // gk, gk).max(axis=(1, 3))


def per_token_cast_to_fp8(x):
    """x fp32 [m, k], k % 128 == 0 -> (codes uint8 [m, k], scales fp32 [m, k/128])."""
    x = np.asarray(x, dtype=np.float32)
    m, k = x.shape
    assert k % 128 == 0
    amax = np.maximum(_grouped_amax(x, 1, 128), np.float32(1e-4)).astype(np.float32)       # [m, k/128]
    q = x.reshape(m, k // 128, 128) * (np.float32(FP8_MAX) / amax)[:, :, None]
    return e4m3fn_encode(q.reshape(m, k)), (amax / np.float32(FP8_MAX)).astype(np.float32)


def per_block_cast_to_fp8(w):
    """w fp32 [n, k], k % 128 == 0 -> (codes uint8 [n, k], scales fp32 [ceil(n/128), k/128]); a ragged last
    row block is scaled by the amax of the rows that exist."""
    w = np.asarray(w, dtype=np.float32)
    n, k = w.shape
    assert k % 128 == 0
    n_pad = -(-n // 128) * 128
    wp = np.zeros((n_pad, k), dtype=np.float32)
    wp[:n] = w
    amax = np.maximum(_grouped_amax(wp, 128, 128), np.float32(1e-4)).astype(np.float32)    # [n/128, k/128]
    q = wp.reshape(n_pad // 128, 128, k // 128, 128) * (np.float32(FP8_MAX) / amax)[:, None, :, None]
    return e4m3fn_encode(q.reshape(n_pad, k)[:n]), (amax / np.float32(FP8_MAX)).astype(np.float32)


def dequant_lhs(codes, scales) -> np.ndarray:
    return e4m3fn_decode(codes) * np.repeat(np.asarray(scales, dtype=np.float32), 128, axis=1)


def dequant_rhs(codes, scales) -> np.ndarray:
    n = np.asarray(codes).shape[0]
    s = np.repeat(np.repeat(np.asarray(scales, dtype=np.float32), 128, axis=0)[:n], 128, axis=1)
    return e4m3fn_decode(codes) * s


# ----------------------------------------------------------------------------- GEMMs
def gemm_bf16_tn_ref(a, b, dtype=np.float32) -> np.ndarray:
    """a [m,k], b [n,k] given as fp32 arrays holding bf16-representable values (or any fp32): a @ b.T."""
    return np.asarray(a, dtype=dtype) @ np.asarray(b, dtype=dtype).T


def gemm_float_nt_ref(a, b, c=None, alpha=1.0, beta=0.0) -> np.ndarray:
    """a [m,k], b [n,k], c [m,n] (logical arrays, any storage order): alpha * a @ b.T + beta * c in fp64; beta == 0
    ignores c."""
    out = float(alpha) * (np.asarray(a, dtype=np.float64) @ np.asarray(b, dtype=np.float64).T)
    if beta != 0.0:
        out = out + float(beta) * np.asarray(c, dtype=np.float64)
    return out


def gemm_fp8_block_scaled_ref(lhs, lhs_scales, rhs, rhs_scales, dtype=np.float32) -> np.ndarray:
    """matmul of the dequantised operands (the parity definition for the FP8 path)."""
    return dequant_lhs(lhs, lhs_scales).astype(dtype) @ dequant_rhs(rhs, rhs_scales).astype(dtype).T


def gemm_fp8_blockwise_f32(lhs, lhs_scales, rhs, rhs_scales) -> np.ndarray:
    """Same value, evaluated the way a block-scaled kernel does: an unscaled fp32 partial product per 128-deep
    K block, folded in as acc += (sA * sB) * partial."""
    a, b = e4m3fn_decode(lhs), e4m3fn_decode(rhs)
    m, k = a.shape
    n = b.shape[0]
    sa = np.asarray(lhs_scales, dtype=np.float32)
    sb = np.repeat(np.asarray(rhs_scales, dtype=np.float32), 128, axis=0)[:n]          # [n, k/128]
    acc = np.zeros((m, n), dtype=np.float32)
    for kb in range(k // 128):
        part = a[:, kb * 128:(kb + 1) * 128] @ b[:, kb * 128:(kb + 1) * 128].T
        acc += part * (sa[:, kb][:, None] * sb[:, kb][None, :])
    return acc


def m_grouped_gemm_contiguous_ref(lhs, lhs_scales, rhs, rhs_scales, m_indices, out_init=None, dtype=np.float32) -> np.ndarray:
    """lhs [m, k] codes, lhs_scales [m, k/128]; rhs [G, n, k] codes, rhs_scales [G, ceil(n/128), k/128];
    m_indices [m] ints: out[i] = row i of the block-scaled product with group m_indices[i]'s weights; rows with a
    negative index keep `out_init` (zeros if not given)."""
    lhs, rhs, m_indices = np.asarray(lhs), np.asarray(rhs), np.asarray(m_indices)
    m, n = lhs.shape[0], rhs.shape[1]
    out = np.zeros((m, n), dtype=dtype) if out_init is None else np.array(out_init, dtype=dtype)
    for g in range(rhs.shape[0]):
        rows = np.nonzero(m_indices == g)[0]
        if rows.size:
            out[rows] = gemm_fp8_block_scaled_ref(lhs[rows], np.asarray(lhs_scales)[rows], rhs[g], np.asarray(rhs_scales)[g], dtype)
    return out


def m_grouped_gemm_masked_ref(lhs, lhs_scales, rhs, rhs_scales, masked_m, out_init=None, dtype=np.float32) -> np.ndarray:
    """lhs [G, m_max, k], lhs_scales [G, m_max, k/128], rhs [G, n, k], rhs_scales [G, ceil(n/128), k/128], masked_m [G]:
    out[g, :masked_m[g]] = block-scaled product of group g's first masked_m[g] rows; other rows keep `out_init`."""
    lhs, rhs = np.asarray(lhs), np.asarray(rhs)
    G, m_max, n = lhs.shape[0], lhs.shape[1], rhs.shape[1]
    out = np.zeros((G, m_max, n), dtype=dtype) if out_init is None else np.array(out_init, dtype=dtype)
    for g in range(G):
        r = int(min(max(int(np.asarray(masked_m)[g]), 0), m_max))
        if r:
            out[g, :r] = gemm_fp8_block_scaled_ref(lhs[g, :r], np.asarray(lhs_scales)[g, :r], rhs[g], np.asarray(rhs_scales)[g], dtype)
    return out
