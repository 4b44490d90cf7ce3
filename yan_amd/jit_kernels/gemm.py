"""FP8 e4m3 block-scaled GEMM, DeepGEMM convention: per-token 1x128 activation scales, 128x128 weight scales.

The reference ships only the JIT template of this op (`yan/jit_kernels/gemm.py:8-31`: keys `N, K, BLOCK_M,
BLOCK_N, NUM_STAGES, NUM_TMA_MULTICAST`; run-time names `lhs, lhs_scales, rhs, rhs_scales, out, m, stream,
num_sms, smem_size`) and no Python entry. `template` and `arg_defs` below keep exactly those keys and names; TMA
descriptors have no gfx950 counterpart, so the operands go to `Gemm::run` as plain pointers. Activation scales that are
not token-contiguous (row-major, say) run through `strided_template`, which takes their two strides as extra arguments,
so no layout needs a transposing copy.

    out[i, j] = bf16( sum_kb lhs_scales[i, kb] * rhs_scales[j // 128, kb]
                              * sum_{t < 128} f32(lhs[i, 128 kb + t]) * f32(rhs[j, 128 kb + t]) )
"""
import functools
from typing import Tuple

import torch

from .heuristics import (get_best_fp8_config, get_fp8_num_stages, get_fp8_tile_space, get_skinny_fp8_config,
                         get_split_k_fp8_config, tuning_enabled)
from .split_k import SPLIT_K_COUNTER_BYTES, SPLIT_K_WORKSPACE_BYTES, split_k_launch_failed, split_k_workspace
from .tuner import FrozenKeys, jit_tuner
from .utils import current_raw_stream, get_num_sms, ceil_div, get_col_major_tensor, scales_for_kernel

# C++ code templates
includes = ('"gemm/fp8_gemm.hpp"', '"gemm/fp8_gemm_skinny.hpp"')

_keys_block = """
using namespace yan;

// Templated args from Python JIT call
constexpr auto N = {N}, K = {K};
constexpr auto BLOCK_M = {BLOCK_M};
constexpr auto BLOCK_N = {BLOCK_N};
constexpr auto kNumStages = {NUM_STAGES};
constexpr auto kNumTMAMulticast = {NUM_TMA_MULTICAST};
"""
# Activation scales as DeepGEMM-style callers hand them over (`get_col_major_tensor`): element (i, kb) at kb * m + i.
_token_contiguous_scales = """
// Token-contiguous activation scales
const int lhs_scales_stride_m = 1, lhs_scales_stride_k = m;
"""
_tiled_launch = """
// Make a templated GEMM
using GemmType = Gemm<N, K, BLOCK_M, BLOCK_N, 128, 1, kNumStages, kNumTMAMulticast, GemmType::Normal>;

// Launch kernel
__return_code = static_cast<int>(GemmType::run(out, lhs, lhs_scales, lhs_scales_stride_m, lhs_scales_stride_k,
                                               rhs, rhs_scales, m, stream, num_sms, smem_size));
"""
# A handful of activation rows: BLOCK_M / 16 activation atoms and 16 weight rows per workgroup, the K blocks of a
# workgroup shared out over NUM_WAVES waves; no LDS staging, NUM_STAGES is the per-wave load depth's name only.
_skinny_launch = """static_assert(BLOCK_N == 16 && BLOCK_M % 16 == 0);

// Launch kernel
__return_code = static_cast<int>(launch_fp8_skinny<N, K, BLOCK_M / 16, {NUM_WAVES}>(
    out, lhs, lhs_scales, lhs_scales_stride_m, lhs_scales_stride_k, rhs, rhs_scales, m, N, K, stream));
"""

# K split over SPLIT_K workgroups per tile; the parts meet in `workspace` (Gemm::run_split_k in gemm/fp8_gemm.hpp).
_split_k_launch = """
// Make a templated GEMM
using GemmType = Gemm<N, K, BLOCK_M, BLOCK_N, 128, 1, kNumStages, kNumTMAMulticast, GemmType::Normal>;

// Launch kernel
__return_code = static_cast<int>(GemmType::run_split_k<{SPLIT_K}>(out, lhs, lhs_scales, lhs_scales_stride_m, lhs_scales_stride_k,
                                                                  rhs, rhs_scales, m, N, K, stream, workspace, workspace_bytes));
"""

# bf16 activations: the quantiser and the GEMM enqueued by one `launch` (gemm_bf16_fp8_bf16_nt below). The codes and their
# token-contiguous scales go to the scratch area behind the split-K workspace proper; the GEMM launch is one of the three above.
_cast_prologue = """
// Quantise the activations into the scratch area behind the split-K workspace: codes [m, K], then scales with element (i, kb) at kb * m + i
static_assert(K % 128 == 0);
if (scratch_bytes < int64_t(m) * K + 256 + int64_t(m) * (K / 128) * 4) { __return_code = static_cast<int>(hipErrorInvalidValue); return; }
uint8_t* scratch = buffer + {SCRATCH_OFFSET};
__hip_fp8_e4m3* lhs = reinterpret_cast<__hip_fp8_e4m3*>(scratch);
float* lhs_scales = reinterpret_cast<float*>(scratch + ((int64_t(m) * K + 255) / 256) * 256);
__return_code = static_cast<int>(launch_per_token_cast(reinterpret_cast<const __bf16*>(x), lhs, lhs_scales, 1, m, m, K, stream));
if (__return_code != 0) return;
"""
_cast_arg_defs_head = (('x', torch.bfloat16), ('buffer', torch.uint8), ('scratch_bytes', int))
cast_includes = includes + ('"gemm/fp8_cast.hpp"', )

# The reference's keys and run-time names, nothing else (yan/jit_kernels/gemm.py:9-30): code that formats this template
# with `N, K, BLOCK_M, BLOCK_N, NUM_STAGES, NUM_TMA_MULTICAST` and builds it with `arg_defs` gets the kernel for
# token-contiguous activation scales.
template = _keys_block + _token_contiguous_scales + _tiled_launch
arg_defs = (('lhs', torch.float8_e4m3fn), ('lhs_scales', torch.float),
            ('rhs', torch.float8_e4m3fn), ('rhs_scales', torch.float),
            ('out', torch.bfloat16), ('m', int),
            ('stream', torch.cuda.Stream), ('num_sms', int), ('smem_size', int))
# Any other strided layout of the activation scales (row-major included) runs without a transposing copy: the same
# kernels with the two strides, in elements, as two more run-time arguments.
strided_template = _keys_block + _tiled_launch
strided_arg_defs = arg_defs + (('lhs_scales_stride_m', int), ('lhs_scales_stride_k', int))
skinny_template = _keys_block + _token_contiguous_scales + _skinny_launch
skinny_strided_template = _keys_block + _skinny_launch
# Split-K kernels take their workspace as two more arguments (in front of the strides, when those are passed).
split_k_template = _keys_block + _token_contiguous_scales + _split_k_launch
split_k_strided_template = _keys_block + _split_k_launch
split_k_arg_defs = arg_defs + (('workspace', torch.uint8), ('workspace_bytes', int))
split_k_strided_arg_defs = split_k_arg_defs + (('lhs_scales_stride_m', int), ('lhs_scales_stride_k', int))

@functools.lru_cache(maxsize=None)
def fp8_kernel_plan(m: int, n: int, k: int, num_cus: int, token_contiguous_scales: bool = True):
    """(name, keys, arg_defs, smem_size, template) of the JIT kernel a call with these sizes uses when K is not split
    (`fp8_split_k_plan` says when it is); needs no GPU."""
    defs = arg_defs if token_contiguous_scales else strided_arg_defs
    # the tuner memoises per (name, keys): the two argument lists need two names
    name = 'gemm_fp8_fp8_bf16_nt' if token_contiguous_scales else 'gemm_fp8_fp8_bf16_nt_strided'
    skinny_atoms = get_skinny_fp8_config(m, n, k, num_cus)
    if skinny_atoms:
        keys = FrozenKeys({'N': n, 'K': k, 'BLOCK_M': 16 * skinny_atoms, 'BLOCK_N': 16, 'NUM_STAGES': 4, 'NUM_TMA_MULTICAST': 1,
                'NUM_WAVES': 8})
        return (name, keys, defs, 8 * skinny_atoms * 64 * 16,
                skinny_template if token_contiguous_scales else skinny_strided_template)
    block_m, block_n = get_best_fp8_config(m, n, k, num_cus)
    keys = FrozenKeys({'N': n, 'K': k, 'BLOCK_M': block_m, 'BLOCK_N': block_n, 'NUM_STAGES': get_fp8_num_stages(block_m, block_n),
            'NUM_TMA_MULTICAST': 1})
    smem_size = keys['NUM_STAGES'] * (block_m + block_n) * 128
    return name, keys, defs, smem_size, template if token_contiguous_scales else strided_template


@functools.lru_cache(maxsize=None)
def fp8_split_k_plan(m: int, n: int, k: int, num_cus: int, token_contiguous_scales: bool = True):
    """(name, keys, arg_defs, template) of the split-K kernel a call with these sizes uses, or None when K is not split
    (`get_split_k_fp8_config`); needs no GPU."""
    plan = get_split_k_fp8_config(m, n, k, num_cus)
    if plan is None:
        return None
    block_m, block_n, split_k = plan
    keys = FrozenKeys({'N': n, 'K': k, 'BLOCK_M': block_m, 'BLOCK_N': block_n, 'NUM_STAGES': get_fp8_num_stages(block_m, block_n),
                       'NUM_TMA_MULTICAST': 1, 'SPLIT_K': split_k})
    if token_contiguous_scales:
        return 'gemm_fp8_fp8_bf16_nt_split_k', keys, split_k_arg_defs, split_k_template
    return 'gemm_fp8_fp8_bf16_nt_split_k_strided', keys, split_k_strided_arg_defs, split_k_strided_template


@functools.lru_cache(maxsize=None)
def fp8_tuning_plan(m: int, n: int, k: int, num_cus: int, token_contiguous_scales: bool = True):
    """(name, keys, space, arg_defs, template) for empirical tile selection among the cost model's three best tiles of
    the tiled kernel (`m` joins the keys as the tuner's memo key), or None when the weight-streaming kernel runs."""
    if get_skinny_fp8_config(m, n, k, num_cus):
        return None
    space = tuple({'BLOCK_M': bm, 'BLOCK_N': bn, 'NUM_STAGES': get_fp8_num_stages(bm, bn)}
                  for bm, bn in get_fp8_tile_space(m, n, k, num_cus))
    keys = FrozenKeys({'M': m, 'N': n, 'K': k, 'NUM_TMA_MULTICAST': 1})
    if token_contiguous_scales:
        return 'gemm_fp8_fp8_bf16_nt', keys, space, arg_defs, template
    return 'gemm_fp8_fp8_bf16_nt_strided', keys, space, strided_arg_defs, strided_template


def gemm_fp8_fp8_bf16_nt(lhs: Tuple[torch.Tensor, torch.Tensor],
                         rhs: Tuple[torch.Tensor, torch.Tensor],
                         out: torch.Tensor) -> None:
    """
    lhs: (e4m3fn `[m, k]` row-major, fp32 scales `[m, ceil(k/128)]` in any strided layout)
    rhs: (e4m3fn `[n, k]` row-major, fp32 scales `[ceil(n/128), ceil(k/128)]` row-major)
    out: bf16 `[m, n]` row-major, written in place; the call is asynchronous on the current stream.
    Requires k % 128 == 0 and n % 4 == 0; m is arbitrary.
    """
    lhs, lhs_scales = lhs
    rhs, rhs_scales = rhs
    m, k = lhs.shape
    n, k_ = rhs.shape
    m_, n_ = out.shape

    assert n % 4 == 0 and k % 128 == 0
    assert m == m_ and n == n_ and k == k_
    assert lhs_scales.shape == (m, ceil_div(k, 128))
    assert rhs_scales.shape == (ceil_div(n, 128), ceil_div(k, 128))
    assert lhs.dtype == torch.float8_e4m3fn and lhs_scales.dtype == torch.float32
    assert rhs.dtype == torch.float8_e4m3fn and rhs_scales.dtype == torch.float32
    assert out.dtype == torch.bfloat16
    assert lhs.is_contiguous() and rhs.is_contiguous() and out.is_contiguous() and rhs_scales.is_contiguous()

    # Do nothing if `m` is zero
    if m == 0:
        return

    num_sms = get_num_sms()
    lhs_scales = scales_for_kernel(lhs_scales, 2.0 * m * n * k)
    stride_m, stride_k = lhs_scales.stride()
    token_contiguous = (m == 1 or stride_m == 1) and (lhs_scales.size(1) == 1 or stride_k == m)
    name, keys, defs, smem_size, code_template = fp8_kernel_plan(m, n, k, num_sms, token_contiguous)
    stream = current_raw_stream()
    args = (lhs, lhs_scales, rhs, rhs_scales, out, m, stream, num_sms, smem_size)
    space, workspace_token = (), None
    if tuning_enabled():
        tuning = fp8_tuning_plan(m, n, k, num_sms, token_contiguous)
        if tuning is not None:
            name, keys, space, defs, code_template = tuning
    else:
        split = fp8_split_k_plan(m, n, k, num_sms, token_contiguous)
        if split is not None:
            workspace, workspace_token = split_k_workspace(out.device, stream)
            if workspace is not None:
                name, keys, defs, code_template = split
                args += (workspace, SPLIT_K_WORKSPACE_BYTES)
    if not token_contiguous:
        args += (stride_m, stride_k)
    runtime = jit_tuner.compile_and_tune(name=name, keys=keys, space=space, includes=includes,
                                         arg_defs=defs, template=code_template, args=args)
    rc = runtime(*args)
    if rc != 0 and workspace_token is not None:
        split_k_launch_failed(workspace_token)
    assert rc == 0, f'{name} failed with HIP error {rc}'


# Scratch of the chained entry: behind the 16 MB of the split-K workspace, room for the codes and scales of up to
# CAST_SCRATCH_BYTES / (k + k / 32) rows (64 rows of K = 65536, 1024 rows of K = 4096).
CAST_SCRATCH_BYTES = 4 << 20


@functools.lru_cache(maxsize=None)
def fp8_cast_chain_plan(m: int, n: int, k: int, num_cus: int, split_k_allowed: bool = True):
    """(name, keys, arg_defs, template, smem_size) of the kernel.so whose `launch` enqueues the per-token quantiser and then the
    GEMM the FP8 entry would run for these sizes (split-K plan, weight-streaming kernel or tiles), or None when the codes
    and scales of `m` rows do not fit the scratch area; needs no GPU."""
    if m <= 0 or m * k + m * (k // 128) * 4 + 256 > CAST_SCRATCH_BYTES:
        return None
    split = fp8_split_k_plan(m, n, k, num_cus, True) if split_k_allowed else None
    if split is not None:
        _, keys, defs, code_template = split
        smem_size = keys['NUM_STAGES'] * (keys['BLOCK_M'] + keys['BLOCK_N']) * 128
    else:
        _, keys, defs, smem_size, code_template = fp8_kernel_plan(m, n, k, num_cus, True)
    # the inner templates start with the keys block and the stride definitions; the prologue goes between those and the launch
    head = _keys_block + _token_contiguous_scales
    assert code_template.startswith(head)
    chained = head + _cast_prologue + code_template[len(head):]
    inner = tuple(d for d in defs if d[0] not in ('lhs', 'lhs_scales'))
    keys = FrozenKeys({**keys, 'SCRATCH_OFFSET': SPLIT_K_WORKSPACE_BYTES})
    return 'gemm_bf16_fp8_bf16_nt', keys, _cast_arg_defs_head + inner, chained, smem_size


def gemm_bf16_fp8_bf16_nt(x: torch.Tensor, rhs: Tuple[torch.Tensor, torch.Tensor], out: torch.Tensor) -> None:
    """`gemm_fp8_fp8_bf16_nt(per_token_cast_to_fp8(x, col_major_scales=True), rhs, out)` for bf16 activations `x` `[m, k]`,
    bit for bit (the same two kernels), as ONE call: one trip through Python and one `launch`, which enqueues the quantiser and
    the GEMM back to back; the codes and scales live in scratch memory the entry keeps per stream, so nothing is allocated
    per call. What a decode step saves is host time: two entry calls cost 18-22 us of Python, which is more than both
    kernels take on the device (64 x 4096 x 7168: 21.7 -> about 13 us call to call). The reference names only the GEMM's
    operands (`yan/jit_kernels/gemm.py:23-30`); the chain of torch ops its callers put in front of it is what this takes
    out of the decode latency. Quantising inside the GEMM kernel itself was built and measured, and is slower than the two
    kernels: every one of the 64 workgroups that share a K range repeats the quantisation of its 64 x 1792 activations,
    9.6 us of vector arithmetic per workgroup against 2.5 us for the quantiser kernel spread over the chip (21.5 us in one
    kernel against 3 + 9.7 us in two; same bits). Problems whose codes do not fit the scratch area (or with
    `YAN_SPLIT_K=0`, which means no memory kept by the entries) run the two entries one after the other."""
    from .fp8_cast import per_token_cast_to_fp8
    from .split_k import split_k_enabled
    rhs_q, rhs_scales = rhs
    m, k = x.shape
    n, k_ = rhs_q.shape
    assert x.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and rhs_q.dtype == torch.float8_e4m3fn and rhs_scales.dtype == torch.float32
    assert out.shape == (m, n) and k == k_ and n % 4 == 0 and k % 128 == 0
    assert rhs_scales.shape == (ceil_div(n, 128), ceil_div(k, 128))
    assert x.is_contiguous() and rhs_q.is_contiguous() and out.is_contiguous() and rhs_scales.is_contiguous()
    if m == 0:
        return
    num_sms = get_num_sms()
    plan = fp8_cast_chain_plan(m, n, k, num_sms) if split_k_enabled() and not tuning_enabled() else None
    if plan is None:
        gemm_fp8_fp8_bf16_nt(per_token_cast_to_fp8(x, col_major_scales=True), rhs, out)
        return
    name, keys, defs, code_template, smem_size = plan
    stream = current_raw_stream()
    workspace, workspace_token = split_k_workspace(out.device, stream)
    values = {'x': x, 'buffer': workspace, 'scratch_bytes': CAST_SCRATCH_BYTES, 'rhs': rhs_q, 'rhs_scales': rhs_scales,
              'out': out, 'm': m, 'stream': stream, 'num_sms': num_sms, 'smem_size': smem_size, 'workspace': workspace,
              'workspace_bytes': SPLIT_K_WORKSPACE_BYTES}
    args = tuple(values[d[0]] for d in defs)
    runtime = jit_tuner.compile_and_tune(name=name, keys=keys, space=(), includes=cast_includes, arg_defs=defs, template=code_template, args=args)
    rc = runtime(*args)
    if rc != 0:
        split_k_launch_failed(workspace_token)
    assert rc == 0, f'{name} failed with HIP error {rc}'
