"""ctypes binding of the ahead-of-time C-ABI library (include/yan_gemm.h). There is no fallback: if
libyan_gemm.so has not been built (`python yan_amd/csrc/build.py`), loading raises."""
import ctypes
import os

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'csrc', 'libyan_gemm.so')
_lib = None

SYMBOLS = ('yan_gemm_bf16_tn', 'yan_gemm_fp16_tn', 'yan_gemm_float_nt', 'yan_gemm_fp8_fp8_bf16_nt', 'yan_m_grouped_gemm_fp8_fp8_bf16_nt_contiguous',
           'yan_m_grouped_gemm_fp8_fp8_bf16_nt_masked', 'yan_per_token_cast_to_fp8', 'yan_per_block_cast_to_fp8',
           'yan_gemm_select_tile', 'yan_gemm_fp8_fp8_bf16_nt_split_k', 'yan_gemm_fp8_fp8_bf16_nt_static', 'yan_gemm_bf16_tn_split_k', 'yan_gemm_fp16_tn_split_k', 'yan_gemm_select_split_k',
           'yan_gemm_split_k_reset', 'yan_gemm_split_k_workspace_bytes', 'yan_gemm_split_k_counter_bytes', 'yan_gemm_version')


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(f'{_LIB_PATH} is missing: build it with `python yan_amd/csrc/build.py`')
        lib = ctypes.CDLL(_LIB_PATH)
        vp, ci, ll = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong
        lib.yan_gemm_bf16_tn.argtypes = lib.yan_gemm_fp16_tn.argtypes = [ci, ci, ci, vp, vp, vp, vp]
        lib.yan_gemm_float_nt.argtypes = [ci, ci, ci, ctypes.c_float, vp, ci, vp, ci, ctypes.c_float, vp, ci, vp]
        lib.yan_gemm_fp8_fp8_bf16_nt.argtypes = lib.yan_gemm_fp8_fp8_bf16_nt_static.argtypes = [vp, vp, ll, ll, vp, vp, vp, ci, ci, ci, vp, ci]
        lib.yan_gemm_select_tile.argtypes = [ci, ci, ci, ci, ci, ctypes.POINTER(ci), ctypes.POINTER(ci)]
        lib.yan_m_grouped_gemm_fp8_fp8_bf16_nt_contiguous.argtypes = [vp, vp, ll, ll, vp, vp, vp, vp, ci, ci, ci, ci, vp, ci]
        lib.yan_m_grouped_gemm_fp8_fp8_bf16_nt_masked.argtypes = [vp, vp, ll, ll, ll, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp, ci]
        lib.yan_per_token_cast_to_fp8.argtypes = [vp, ci, vp, vp, ll, ll, ci, ci, vp]
        lib.yan_per_block_cast_to_fp8.argtypes = [vp, ci, vp, vp, ci, ci, vp]
        lib.yan_gemm_fp8_fp8_bf16_nt_split_k.argtypes = [vp, vp, ll, ll, vp, vp, vp, ci, ci, ci, vp, ci, vp, ll]
        lib.yan_gemm_select_split_k.argtypes = [ci, ci, ci, ci, ci, ctypes.POINTER(ci), ctypes.POINTER(ci), ctypes.POINTER(ci)]
        lib.yan_gemm_bf16_tn_split_k.argtypes = lib.yan_gemm_fp16_tn_split_k.argtypes = [ci, ci, ci, vp, vp, vp, vp, vp, ll]
        lib.yan_gemm_split_k_reset.argtypes = [vp, vp]
        lib.yan_gemm_split_k_workspace_bytes.argtypes = lib.yan_gemm_split_k_counter_bytes.argtypes = []
        for name in SYMBOLS[:-1]:
            getattr(lib, name).restype = ci
        lib.yan_gemm_split_k_workspace_bytes.restype = lib.yan_gemm_split_k_counter_bytes.restype = ll
        lib.yan_gemm_version.restype = ctypes.c_char_p
        _lib = lib
    return _lib


def _stream_handle():
    from .jit_kernels.utils import current_raw_stream
    return ctypes.c_void_p(current_raw_stream())


def gemm_bf16_tn(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor) -> int:
    (m, k), n = a.shape, b.shape[0]
    return load().yan_gemm_bf16_tn(m, n, k, a.data_ptr(), b.data_ptr(), c.data_ptr(), _stream_handle())


def gemm_fp16_tn(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor) -> int:
    (m, k), n = a.shape, b.shape[0]
    return load().yan_gemm_fp16_tn(m, n, k, a.data_ptr(), b.data_ptr(), c.data_ptr(), _stream_handle())


def gemm_float_nt(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor, alpha: float = 1.0, beta: float = 0.0) -> int:
    """`a` [m, k] and `b` [n, k] with their first dimension contiguous, `c` [m, n] row-major."""
    (m, k), n = a.shape, b.shape[0]
    lda = a.stride(1) if k > 1 else m
    ldb = b.stride(1) if k > 1 else n
    return load().yan_gemm_float_nt(m, n, k, alpha, a.data_ptr(), lda, b.data_ptr(), ldb, beta, c.data_ptr(), c.stride(0),
                                    _stream_handle())


def gemm_fp8_fp8_bf16_nt(lhs, rhs, out: torch.Tensor, num_sms: int = 0) -> int:
    (a8, sa), (b8, sb) = lhs, rhs
    (m, k), n = a8.shape, b8.shape[0]
    return load().yan_gemm_fp8_fp8_bf16_nt(a8.data_ptr(), sa.data_ptr(), sa.stride(0), sa.stride(1), b8.data_ptr(),
                                           sb.data_ptr(), out.data_ptr(), m, n, k, _stream_handle(), num_sms)


def split_k_workspace(device='cuda') -> torch.Tensor:
    """A zero-filled workspace for the split-K entry points, of the size the library asks for."""
    return torch.zeros(load().yan_gemm_split_k_workspace_bytes(), dtype=torch.uint8, device=device)


def gemm_fp8_fp8_bf16_nt_split_k(lhs, rhs, out: torch.Tensor, workspace: torch.Tensor, num_sms: int = 0) -> int:
    (a8, sa), (b8, sb) = lhs, rhs
    (m, k), n = a8.shape, b8.shape[0]
    return load().yan_gemm_fp8_fp8_bf16_nt_split_k(a8.data_ptr(), sa.data_ptr(), sa.stride(0), sa.stride(1), b8.data_ptr(),
                                                   sb.data_ptr(), out.data_ptr(), m, n, k, _stream_handle(), num_sms,
                                                   workspace.data_ptr(), workspace.numel() * workspace.element_size())


def gemm_fp8_fp8_bf16_nt_static(lhs, rhs, out: torch.Tensor, num_sms: int = 0) -> int:
    """The split-K GEMM on the library's own device array: nothing is allocated."""
    (a8, sa), (b8, sb) = lhs, rhs
    (m, k), n = a8.shape, b8.shape[0]
    return load().yan_gemm_fp8_fp8_bf16_nt_static(a8.data_ptr(), sa.data_ptr(), sa.stride(0), sa.stride(1), b8.data_ptr(),
                                                  sb.data_ptr(), out.data_ptr(), m, n, k, _stream_handle(), num_sms)


def split_k_reset(workspace: torch.Tensor = None) -> int:
    """Arrival counters of `workspace` (None: the library's own array on the current GPU) back to zero, on the current stream."""
    return load().yan_gemm_split_k_reset(None if workspace is None else workspace.data_ptr(), _stream_handle())


def gemm_bf16_tn_split_k(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor, workspace: torch.Tensor) -> int:
    (m, k), n = a.shape, b.shape[0]
    fn = load().yan_gemm_bf16_tn_split_k if a.dtype == torch.bfloat16 else load().yan_gemm_fp16_tn_split_k
    return fn(m, n, k, a.data_ptr(), b.data_ptr(), c.data_ptr(), _stream_handle(), workspace.data_ptr(),
              workspace.numel() * workspace.element_size())


def select_split_k(m: int, n: int, k: int, num_cus: int, op: int = 1):
    """(BLOCK_M, BLOCK_N, SPLIT_K) of the library's split-K plan (op 0: dense, 1: FP8), or None when K is not split."""
    bm, bn, split = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    assert load().yan_gemm_select_split_k(op, m, n, k, num_cus, ctypes.byref(bm), ctypes.byref(bn), ctypes.byref(split)) == 0
    return (bm.value, bn.value, split.value) if split.value > 1 else None


def m_grouped_gemm_fp8_fp8_bf16_nt_contiguous(lhs, rhs, out: torch.Tensor, m_indices: torch.Tensor, num_sms: int = 0) -> int:
    (a8, sa), (b8, sb) = lhs, rhs
    (m, k), (groups, n, _) = a8.shape, b8.shape
    return load().yan_m_grouped_gemm_fp8_fp8_bf16_nt_contiguous(
        a8.data_ptr(), sa.data_ptr(), sa.stride(0), sa.stride(1), b8.data_ptr(), sb.data_ptr(), out.data_ptr(),
        m_indices.data_ptr(), groups, m, n, k, _stream_handle(), num_sms)


def m_grouped_gemm_fp8_fp8_bf16_nt_masked(lhs, rhs, out: torch.Tensor, masked_m: torch.Tensor, expected_m: int,
                                          num_sms: int = 0) -> int:
    (a8, sa), (b8, sb) = lhs, rhs
    (groups, m_max, k), n = a8.shape, b8.shape[1]
    return load().yan_m_grouped_gemm_fp8_fp8_bf16_nt_masked(
        a8.data_ptr(), sa.data_ptr(), sa.stride(0), sa.stride(1), sa.stride(2), b8.data_ptr(), sb.data_ptr(),
        out.data_ptr(), masked_m.data_ptr(), groups, m_max, expected_m, n, k, _stream_handle(), num_sms)


def per_token_cast_to_fp8(x: torch.Tensor, q: torch.Tensor, scales: torch.Tensor) -> int:
    m, k = x.shape
    return load().yan_per_token_cast_to_fp8(x.data_ptr(), int(x.dtype == torch.float32), q.data_ptr(), scales.data_ptr(),
                                            scales.stride(0), scales.stride(1), m, k, _stream_handle())


def per_block_cast_to_fp8(w: torch.Tensor, q: torch.Tensor, scales: torch.Tensor) -> int:
    n, k = w.shape
    return load().yan_per_block_cast_to_fp8(w.data_ptr(), int(w.dtype == torch.float32), q.data_ptr(), scales.data_ptr(),
                                            n, k, _stream_handle())


def select_tile(op: int, m: int, n: int, k: int, num_cus: int):
    bm, bn = ctypes.c_int(0), ctypes.c_int(0)
    rc = load().yan_gemm_select_tile(op, m, n, k, num_cus, ctypes.byref(bm), ctypes.byref(bn))
    assert rc == 0
    return bm.value, bn.value
