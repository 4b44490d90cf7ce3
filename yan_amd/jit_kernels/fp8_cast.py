"""Quantisers in front of the block-scaled FP8 GEMM: per-token 1x128 for activations, per-block 128x128 for weights.

The reference names the GEMM's operands (`lhs, lhs_scales, rhs, rhs_scales`, `yan/jit_kernels/gemm.py:23-30`) and has
no code that produces them; callers of this convention build them with a chain of torch ops
(`amax = |x|.view(m, -1, 128).amax(-1).clamp(1e-4)`, `q = (x * (448 / amax)).to(float8_e4m3fn)`, `scale = amax / 448`).
The two entries here do the same arithmetic in one kernel each, one pass over HBM. Both quotients are correctly
rounded fp32 divisions; torch evaluates `448.0 / amax` as `reciprocal(amax) * 448`, which is an ulp away for some
amax and moves a code where `x * factor` lands on a rounding boundary. With true tensor / tensor divisions the torch
chain and these kernels agree bit for bit.
"""
import functools
from typing import Tuple

import torch

from .tuner import FrozenKeys, jit_tuner
from .utils import ceil_div, current_raw_stream

includes = ('"gemm/fp8_cast.hpp"', )

per_token_template = """
using namespace yan;
// Templated args from Python JIT call: source element type {SRC}
__return_code = static_cast<int>(launch_per_token_cast(x, q, scales, scales_stride_m, scales_stride_k, m, k, stream));
"""

per_block_template = """
using namespace yan;
// Templated args from Python JIT call: source element type {SRC}
__return_code = static_cast<int>(launch_per_block_cast(x, q, scales, n, k, stream));
"""


def _src_name(dtype: torch.dtype) -> str:
    assert dtype in (torch.bfloat16, torch.float32), 'the quantisers take bf16 or fp32 sources'
    return 'bf16' if dtype == torch.bfloat16 else 'fp32'


def per_token_arg_defs(dtype: torch.dtype):
    return (('x', dtype), ('q', torch.float8_e4m3fn), ('scales', torch.float), ('scales_stride_m', int),
            ('scales_stride_k', int), ('m', int), ('k', int), ('stream', torch.cuda.Stream))


def per_block_arg_defs(dtype: torch.dtype):
    return (('x', dtype), ('q', torch.float8_e4m3fn), ('scales', torch.float), ('n', int), ('k', int),
            ('stream', torch.cuda.Stream))


@functools.lru_cache(maxsize=None)
def cast_kernel_plan(kind: str, dtype: torch.dtype):
    """(name, keys, arg_defs, template) of the JIT kernel behind a quantiser; needs no GPU."""
    keys = FrozenKeys({'SRC': _src_name(dtype)})
    if kind == 'per_token':
        return 'per_token_cast_to_fp8', keys, per_token_arg_defs(dtype), per_token_template
    assert kind == 'per_block'
    return 'per_block_cast_to_fp8', keys, per_block_arg_defs(dtype), per_block_template


def per_token_cast_to_fp8(x: torch.Tensor, col_major_scales: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """x `[m, k]` bf16 or fp32, contiguous, k % 128 == 0 -> (e4m3fn `[m, k]`, fp32 scales `[m, k/128]`).
    With `col_major_scales` the scale tensor is laid out token-contiguous (stride(0) == 1), the layout
    `get_col_major_tensor` gives and the GEMM reads fastest; the values are the same."""
    assert x.dim() == 2 and x.size(1) % 128 == 0 and x.is_contiguous()
    m, k = x.shape
    q = torch.empty((m, k), dtype=torch.float8_e4m3fn, device=x.device)
    if col_major_scales:
        scales = torch.empty((k // 128, m), dtype=torch.float32, device=x.device).t()
    else:
        scales = torch.empty((m, k // 128), dtype=torch.float32, device=x.device)
    if m == 0 or k == 0:
        return q, scales
    name, keys, arg_defs, template = cast_kernel_plan('per_token', x.dtype)
    args = (x, q, scales, scales.stride(0), scales.stride(1), m, k, current_raw_stream())
    runtime = jit_tuner.compile_and_tune(name=name, keys=keys, space=(), includes=includes, arg_defs=arg_defs,
                                         template=template, args=args)
    rc = runtime(*args)
    assert rc == 0, f'{name} failed with HIP error {rc}'
    return q, scales


def per_block_cast_to_fp8(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """w `[n, k]` bf16 or fp32, contiguous, k % 128 == 0 -> (e4m3fn `[n, k]`, fp32 scales `[ceil(n/128), k/128]`);
    a ragged last block of rows is scaled by the maximum of the rows that exist."""
    assert w.dim() == 2 and w.size(1) % 128 == 0 and w.is_contiguous()
    n, k = w.shape
    q = torch.empty((n, k), dtype=torch.float8_e4m3fn, device=w.device)
    scales = torch.empty((ceil_div(n, 128), k // 128), dtype=torch.float32, device=w.device)
    if n == 0 or k == 0:
        return q, scales
    name, keys, arg_defs, template = cast_kernel_plan('per_block', w.dtype)
    args = (w, q, scales, n, k, current_raw_stream())
    runtime = jit_tuner.compile_and_tune(name=name, keys=keys, space=(), includes=includes, arg_defs=arg_defs,
                                         template=template, args=args)
    rc = runtime(*args)
    assert rc == 0, f'{name} failed with HIP error {rc}'
    return q, scales
