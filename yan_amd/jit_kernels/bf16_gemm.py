"""Dense 16-bit GEMM entry points: `c[m,n] = a[m,k] @ b[n,k]^T`, written in place, returns None.

Same contract as the reference's `gemm_fp16_tn` (`yan/jit_kernels/cute_gemm.py:21-64`): `a` is `[m,k]`, `b` is
`[n,k]`, `c` is `[m,n]`, all row-major on the current device; the call is asynchronous on the current stream;
`m == 0` or `n == 0` returns at once. The reference only has the fp16 flavour and accumulates in fp16; here both
bf16 and fp16 exist and both accumulate in fp32. Keys and argument order of the JIT kernel are the reference's:
keys `BLOCK_M, BLOCK_N, NUM_STAGES`, args `(m, n, k, A, B, C, stream)`. The reference's dense kernel is not persistent and
knows no `num_sms`; here a cap set with `set_num_sms` below the device's compute units becomes one more key, `NUM_SMS`
(0 without a cap), so that the argument list stays the reference's.
"""
import functools

import torch

from .heuristics import (get_best_dense_config, get_dense_num_stages, get_dense_tile_space, get_skinny_dense_config,
                         get_split_k_dense_config, tuning_enabled)
from .split_k import SPLIT_K_WORKSPACE_BYTES, split_k_launch_failed, split_k_workspace
from .tuner import FrozenKeys, jit_tuner
from .utils import current_raw_stream, get_num_sms, get_num_sms_cap

includes = ('"gemm/bf16_gemm.hpp"', )
template = """
// Templated args from Python JIT call
constexpr auto BLOCK_M = {BLOCK_M};
constexpr auto BLOCK_N = {BLOCK_N};
constexpr auto kNumStages = {NUM_STAGES};
constexpr auto kNumSMs = {NUM_SMS};

__return_code = static_cast<int>(gemm_tn<BLOCK_M, BLOCK_N, kNumStages>(m, n, k, A, B, C, stream, kNumSMs));
"""
# K split over SPLIT_K workgroups per tile; the parts meet in `workspace` (launch_dense_split_k in gemm/bf16_gemm.hpp).
split_k_template = """
// Templated args from Python JIT call
constexpr auto BLOCK_M = {BLOCK_M};
constexpr auto BLOCK_N = {BLOCK_N};
constexpr auto kNumStages = {NUM_STAGES};
constexpr auto kSplitK = {SPLIT_K};

__return_code = static_cast<int>(gemm_tn_split_k<BLOCK_M, BLOCK_N, kNumStages, kSplitK>(m, n, k, A, B, C, stream, workspace, workspace_bytes));
"""


def _arg_defs(dtype: torch.dtype):
    return (('m', int), ('n', int), ('k', int), ('A', dtype), ('B', dtype), ('C', dtype), ('stream', torch.cuda.Stream))


def _split_k_arg_defs(dtype: torch.dtype):
    return _arg_defs(dtype) + (('workspace', torch.uint8), ('workspace_bytes', int))


@functools.lru_cache(maxsize=None)
def dense_split_k_plan(m: int, n: int, k: int, dtype: torch.dtype, num_cus: int):
    """(name, keys, arg_defs) of the split-K kernel a call with these sizes uses, or None when K is not split
    (`get_split_k_dense_config`); needs no GPU."""
    plan = get_split_k_dense_config(m, n, k, num_cus)
    if plan is None:
        return None
    block_m, block_n, split_k = plan
    name = 'gemm_bf16_tn_split_k' if dtype == torch.bfloat16 else 'gemm_fp16_tn_split_k'
    keys = FrozenKeys({'BLOCK_M': block_m, 'BLOCK_N': block_n, 'NUM_STAGES': get_dense_num_stages(block_m, block_n), 'SPLIT_K': split_k})
    return name, keys, _split_k_arg_defs(dtype)


@functools.lru_cache(maxsize=None)
def dense_kernel_plan(m: int, n: int, k: int, dtype: torch.dtype, num_cus: int, num_sms_cap: int = 0):
    """(name, keys, arg_defs) of the JIT kernel a call with these sizes uses; needs no GPU. `num_cus` steers the tile
    choice, `num_sms_cap` (0 = none) is the number of workgroups the launch may start."""
    name = 'gemm_bf16_tn' if dtype == torch.bfloat16 else 'gemm_fp16_tn'
    skinny_atoms = get_skinny_dense_config(m, n, k, num_cus)
    if skinny_atoms:
        # the weight-streaming kernel for a handful of rows: BLOCK_N = 16 names it, its n / 16 workgroups are within any cap
        return name, FrozenKeys({'BLOCK_M': 16 * skinny_atoms, 'BLOCK_N': 16, 'NUM_STAGES': 1, 'NUM_SMS': 0}), _arg_defs(dtype)
    block_m, block_n = get_best_dense_config(m, n, k, num_cus)
    keys = FrozenKeys({'BLOCK_M': block_m, 'BLOCK_N': block_n, 'NUM_STAGES': get_dense_num_stages(block_m, block_n), 'NUM_SMS': num_sms_cap})
    return name, keys, _arg_defs(dtype)


@functools.lru_cache(maxsize=None)
def dense_tuning_plan(m: int, n: int, k: int, dtype: torch.dtype, num_cus: int, num_sms_cap: int = 0):
    """(name, keys, space, arg_defs) for empirical tile selection: the shape is the tuner's memo key and the cost
    model's three best tiles are its candidates."""
    name = 'gemm_bf16_tn' if dtype == torch.bfloat16 else 'gemm_fp16_tn'
    space = tuple({'BLOCK_M': bm, 'BLOCK_N': bn, 'NUM_STAGES': get_dense_num_stages(bm, bn)}
                  for bm, bn in get_dense_tile_space(m, n, k, num_cus))
    return name, FrozenKeys({'M': m, 'N': n, 'K': k, 'NUM_SMS': num_sms_cap}), space, _arg_defs(dtype)


def _gemm_16bit_tn(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor, dtype: torch.dtype) -> None:
    m, k = a.shape
    n, k_ = b.shape
    m_, n_ = c.shape
    assert m == m_ and n == n_ and k == k_
    assert a.dtype == dtype and b.dtype == dtype and c.dtype == dtype
    assert a.is_contiguous() and b.is_contiguous() and c.is_contiguous()
    assert n % 4 == 0 and k % 8 == 0, 'n must be a multiple of 4 and k a multiple of 8'
    if m == 0 or n == 0:
        return

    stream = current_raw_stream()
    args = (m, n, k, a, b, c, stream)
    code_template, workspace_token = template, None
    if tuning_enabled() and not get_skinny_dense_config(m, n, k, get_num_sms()):
        name, keys, space, arg_defs = dense_tuning_plan(m, n, k, dtype, get_num_sms(), get_num_sms_cap())
    else:
        (name, keys, arg_defs), space = dense_kernel_plan(m, n, k, dtype, get_num_sms(), get_num_sms_cap()), ()
        split = dense_split_k_plan(m, n, k, dtype, get_num_sms())
        if split is not None:
            workspace, workspace_token = split_k_workspace(c.device, stream)
            if workspace is not None:
                name, keys, arg_defs = split
                code_template = split_k_template
                args += (workspace, SPLIT_K_WORKSPACE_BYTES)
    runtime = jit_tuner.compile_and_tune(name=name, keys=keys, space=space, includes=includes,
                                         arg_defs=arg_defs, template=code_template, args=args)
    rc = runtime(*args)
    if rc != 0 and workspace_token is not None:
        split_k_launch_failed(workspace_token)
    assert rc == 0, f'{name} failed with HIP error {rc}'


def gemm_bf16_tn(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor) -> None:
    _gemm_16bit_tn(a, b, c, torch.bfloat16)


def gemm_fp16_tn(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor) -> None:
    _gemm_16bit_tn(a, b, c, torch.half)


def accuracy_test():
    """The reference's smoke check (`cute_gemm.py:67-86`): seed 42, 4096 x 7168 x 2048, against `a @ b.t()`."""
    from ..utils import calc_diff
    torch.manual_seed(42)
    m, n, k = 4096, 7168, 2048
    for dtype, fn in ((torch.bfloat16, gemm_bf16_tn), (torch.half, gemm_fp16_tn)):
        a = torch.randn(m, k, dtype=dtype, device='cuda')
        b = torch.randn(n, k, dtype=dtype, device='cuda')
        c = torch.zeros(m, n, dtype=dtype, device='cuda')
        fn(a, b, c)
        diff = calc_diff(c, a.float() @ b.float().t())
        print(f'{fn.__name__}: calc_diff = {diff:.3e}')
        assert diff < 1e-5
