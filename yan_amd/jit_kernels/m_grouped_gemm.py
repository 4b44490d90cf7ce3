"""Grouped (mixture-of-experts) FP8 block-scaled GEMMs: every group has its own `[n, k]` weight matrix.

The reference carries the hooks for these and no entry point: `GemmType::{GroupedContiguous, GroupedMasked}` and the
`grouped_layout` argument of its scheduler and kernel (`yan/include/gemm/scheduler.cuh:7-11,31-48`,
`yan/include/gemm/fp8_gemm.cuh:41`), the `kNumGroups` slot of the `Gemm<...>` template its JIT code instantiates
(`yan/jit_kernels/gemm.py:20`), and `get_m_alignment_for_contiguous_layout` (`yan/jit_kernels/utils.py:46-55`).
The two entries below complete them with the calling convention of the DeepGEMM functions those hooks come from.
Scales, dtypes and the arithmetic are those of `gemm_fp8_fp8_bf16_nt`, applied per group.
"""
import functools
from typing import Tuple

import torch

from .gemm import includes
from .heuristics import get_best_grouped_fp8_config, get_contiguous_rows_on_device, get_fp8_num_stages
from .tuner import FrozenKeys, jit_tuner
from .utils import ceil_div, current_raw_stream, get_m_alignment_for_contiguous_layout, get_num_sms, scales_for_kernel

template = """
using namespace yan;

// Templated args from Python JIT call
constexpr auto N = {N}, K = {K};
constexpr auto BLOCK_M = {BLOCK_M};
constexpr auto BLOCK_N = {BLOCK_N};
constexpr auto kNumStages = {NUM_STAGES};
constexpr auto kNumTMAMulticast = {NUM_TMA_MULTICAST};
constexpr auto kNumGroups = {NUM_GROUPS};

// Make a templated grouped GEMM
using GemmType = Gemm<N, K, BLOCK_M, BLOCK_N, 128, kNumGroups, kNumStages, kNumTMAMulticast, GemmType::{GEMM_TYPE}>;

// Launch kernel
__return_code = static_cast<int>(GemmType::run_grouped(out, lhs, lhs_scales, lhs_scales_stride_m, lhs_scales_stride_k,
                                                       lhs_scales_stride_g, rhs, rhs_scales, grouped_layout,
                                                       kNumGroups, m, N, K, stream, num_sms, expected_m));
"""

# Contiguous groups of a few hundred rows: the kernel that holds 256 x 256 and 128 x 256 tiles and picks on the device
# (Gemm::run_grouped_rows_on_device in gemm/fp8_gemm.hpp); same keys and arguments.
rows_on_device_template = template.replace(
    """GemmType::run_grouped(out, lhs, lhs_scales, lhs_scales_stride_m, lhs_scales_stride_k,
                                                       lhs_scales_stride_g, rhs, rhs_scales, grouped_layout,
                                                       kNumGroups, m, N, K, stream, num_sms, expected_m)""",
    """GemmType::run_grouped_rows_on_device(out, lhs, lhs_scales, lhs_scales_stride_m, lhs_scales_stride_k,
                                                                      rhs, rhs_scales, grouped_layout, kNumGroups, m, N, K, stream, num_sms)""")
assert rows_on_device_template != template

arg_defs = (('lhs', torch.float8_e4m3fn), ('lhs_scales', torch.float),
            ('rhs', torch.float8_e4m3fn), ('rhs_scales', torch.float),
            ('out', torch.bfloat16), ('grouped_layout', torch.int), ('m', int),
            ('stream', torch.cuda.Stream), ('num_sms', int), ('smem_size', int),
            ('lhs_scales_stride_m', int), ('lhs_scales_stride_k', int), ('lhs_scales_stride_g', int), ('expected_m', int))


@functools.lru_cache(maxsize=None)
def grouped_kernel_plan(gemm_type: str, num_groups: int, m: int, n: int, k: int, num_cus: int):
    """(name, keys, arg_defs, smem_size) of the JIT kernel of a grouped call; needs no GPU. `m` is the total row count
    for 'GroupedContiguous' and the expected rows per group for 'GroupedMasked'."""
    assert gemm_type in ('GroupedContiguous', 'GroupedMasked')
    if gemm_type == 'GroupedContiguous':
        block_m, block_n = get_best_grouped_fp8_config(m, n, k, num_cus, 1, get_m_alignment_for_contiguous_layout(), num_groups)
        name = 'm_grouped_gemm_fp8_fp8_bf16_nt'
        if get_contiguous_rows_on_device(m, n, k, num_cus, num_groups):
            # both tile heights in one kernel, named by the taller one
            keys = FrozenKeys({'N': n, 'K': k, 'BLOCK_M': 256, 'BLOCK_N': 256, 'NUM_GROUPS': num_groups, 'NUM_STAGES': 2,
                               'NUM_TMA_MULTICAST': 1, 'GEMM_TYPE': gemm_type, 'ROWS': 'picked on the device'})
            return name + '_rows_on_device', keys, arg_defs, 2 * (256 + 256) * 128
    else:
        block_m, block_n = get_best_grouped_fp8_config(m, n, k, num_cus, num_groups)
        name = 'm_grouped_gemm_fp8_fp8_bf16_nt'
    keys = FrozenKeys({'N': n, 'K': k, 'BLOCK_M': block_m, 'BLOCK_N': block_n, 'NUM_GROUPS': num_groups,
            'NUM_STAGES': get_fp8_num_stages(block_m, block_n),
            'NUM_TMA_MULTICAST': 1, 'GEMM_TYPE': gemm_type})
    return name, keys, arg_defs, keys['NUM_STAGES'] * (block_m + block_n) * 128


def _launch(gemm_type, num_groups, plan_m, m, n, k, lhs, lhs_scales, rhs, rhs_scales, out, layout, strides):
    # `strides`: the three strides of the activation scales, then expected_m (masked layout; 0 otherwise)
    num_sms = get_num_sms()
    name, keys, defs, smem_size = grouped_kernel_plan(gemm_type, num_groups, plan_m, n, k, num_sms)
    args = (lhs, lhs_scales, rhs, rhs_scales, out, layout, m, current_raw_stream(), num_sms, smem_size, *strides)
    runtime = jit_tuner.compile_and_tune(name=name, keys=keys, space=(), includes=includes, arg_defs=defs,
                                         template=rows_on_device_template if 'ROWS' in keys else template, args=args)
    rc = runtime(*args)
    assert rc == 0, f'{name} failed with HIP error {rc}'


def m_grouped_gemm_fp8_fp8_bf16_nt_contiguous(lhs: Tuple[torch.Tensor, torch.Tensor],
                                              rhs: Tuple[torch.Tensor, torch.Tensor],
                                              out: torch.Tensor, m_indices: torch.Tensor) -> None:
    """
    The rows of all groups concatenated along m, each group padded to a multiple of
    `get_m_alignment_for_contiguous_layout()` rows.

    lhs: (e4m3fn `[m_sum, k]` row-major, fp32 scales `[m_sum, ceil(k/128)]` in any strided layout)
    rhs: (e4m3fn `[num_groups, n, k]`, fp32 scales `[num_groups, ceil(n/128), ceil(k/128)]`), both contiguous
    out: bf16 `[m_sum, n]`, written in place; rows whose index is negative are left untouched
    m_indices: int32 `[m_sum]`, the group of every row (equal within each aligned block of rows; negative marks a
               block of padding rows that is skipped)
    """
    lhs, lhs_scales = lhs
    rhs, rhs_scales = rhs
    m, k = lhs.shape
    num_groups, n, k_ = rhs.shape
    m_, n_ = out.shape
    m__ = m_indices.numel()

    assert n % 4 == 0 and k % 128 == 0
    assert m == m_ == m__ and n == n_ and k == k_
    assert m % get_m_alignment_for_contiguous_layout() == 0, 'groups must be padded to the contiguous-layout alignment'
    assert lhs_scales.shape == (m, ceil_div(k, 128))
    assert rhs_scales.shape == (num_groups, ceil_div(n, 128), ceil_div(k, 128))
    assert lhs.dtype == torch.float8_e4m3fn and lhs_scales.dtype == torch.float32
    assert rhs.dtype == torch.float8_e4m3fn and rhs_scales.dtype == torch.float32
    assert out.dtype == torch.bfloat16 and m_indices.dtype == torch.int32
    assert lhs.is_contiguous() and rhs.is_contiguous() and rhs_scales.is_contiguous()
    assert out.is_contiguous() and m_indices.is_contiguous()

    if m == 0:
        return
    lhs_scales = scales_for_kernel(lhs_scales, 2.0 * m * n * k)
    _launch('GroupedContiguous', num_groups, m, m, n, k, lhs, lhs_scales, rhs, rhs_scales, out, m_indices,
            (lhs_scales.stride(0), lhs_scales.stride(1), 0, 0))


def m_grouped_gemm_fp8_fp8_bf16_nt_masked(lhs: Tuple[torch.Tensor, torch.Tensor],
                                          rhs: Tuple[torch.Tensor, torch.Tensor],
                                          out: torch.Tensor, masked_m: torch.Tensor, expected_m: int) -> None:
    """
    Every group owns `m_max` rows of which only the first `masked_m[g]` are valid (decode with CUDA-graph-style fixed
    shapes); the other rows of `out` are left untouched.

    lhs: (e4m3fn `[num_groups, m_max, k]` contiguous, fp32 scales `[num_groups, m_max, ceil(k/128)]` in any strided layout)
    rhs: (e4m3fn `[num_groups, n, k]`, fp32 scales `[num_groups, ceil(n/128), ceil(k/128)]`), both contiguous
    out: bf16 `[num_groups, m_max, n]` contiguous
    masked_m: int32 `[num_groups]`; expected_m: a hint for the typical masked_m: it picks the tile and puts the tile rows
              below it first in the launch order; results do not depend on it
    """
    lhs, lhs_scales = lhs
    rhs, rhs_scales = rhs
    num_groups, m, k = lhs.shape
    num_groups_, n, k_ = rhs.shape
    num_groups__, m_, n_ = out.shape
    num_groups___ = masked_m.numel()

    assert n % 4 == 0 and k % 128 == 0
    assert num_groups == num_groups_ == num_groups__ == num_groups___
    assert m == m_ and n == n_ and k == k_ and expected_m > 0
    assert lhs_scales.shape == (num_groups, m, ceil_div(k, 128))
    assert rhs_scales.shape == (num_groups, ceil_div(n, 128), ceil_div(k, 128))
    assert lhs.dtype == torch.float8_e4m3fn and lhs_scales.dtype == torch.float32
    assert rhs.dtype == torch.float8_e4m3fn and rhs_scales.dtype == torch.float32
    assert out.dtype == torch.bfloat16 and masked_m.dtype == torch.int32
    assert lhs.is_contiguous() and rhs.is_contiguous() and rhs_scales.is_contiguous()
    assert out.is_contiguous() and masked_m.is_contiguous()

    if m == 0 or num_groups == 0:
        return
    lhs_scales = scales_for_kernel(lhs_scales, 2.0 * num_groups * min(expected_m, m) * n * k)
    _launch('GroupedMasked', num_groups, min(expected_m, m), m, n, k, lhs, lhs_scales, rhs, rhs_scales, out, masked_m,
            (lhs_scales.stride(1), lhs_scales.stride(2), lhs_scales.stride(0), min(expected_m, m)))
