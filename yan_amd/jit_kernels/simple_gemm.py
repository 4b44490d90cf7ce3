"""fp32 GEMM entry point: `c = alpha * a @ b^T + beta * c`, written in place, returns None.

Same contract as the reference's `gemm_float_nt` (`yan/jit_kernels/simple_gemm.py:18-57`): `a` is `[m, k]` and `b` is
`[n, k]`, both stored with their FIRST dimension contiguous (what `get_col_major_tensor` returns; the reference
passes `ldA = m`, `ldB = n` without looking at the strides), `c` is `[m, n]` row-major, all fp32 on the current
device; `m % 128 == 0` and `n % 64 == 0`; the call is asynchronous on the current stream; `m == 0` or `n == 0` returns
at once. Argument order of the JIT kernel is the reference's: `(m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC, stream)`.
The reference compiles one kernel with a fixed 128 x 64 tile (`keys={}`); here the tile is a key.
"""
import functools

import torch

from .heuristics import get_best_float_config
from .tuner import FrozenKeys, jit_tuner
from .utils import current_raw_stream, get_num_sms

includes = ('"gemm/simple_gemm.hpp"', )
template = """
// Templated args from Python JIT call
constexpr auto BLOCK_M = {BLOCK_M};
constexpr auto BLOCK_N = {BLOCK_N};

__return_code = static_cast<int>(gemm_nt<BLOCK_M, BLOCK_N>(m, n, k,
        alpha,
        static_cast<float const*>(A), ldA,
        static_cast<float const*>(B), ldB,
        beta,
        static_cast<float*>(C), ldC,
        stream));
"""

arg_defs = (('m', int), ('n', int), ('k', int),
            ('alpha', float),
            ('A', torch.float), ('ldA', int),
            ('B', torch.float), ('ldB', int),
            ('beta', float),
            ('C', torch.float), ('ldC', int),
            ('stream', torch.cuda.Stream))


@functools.lru_cache(maxsize=None)
def float_kernel_plan(m: int, n: int, num_cus: int):
    """(name, keys, arg_defs) of the JIT kernel a call with these sizes uses; needs no GPU."""
    block_m, block_n = get_best_float_config(m, n, num_cus)
    return 'gemm_float_nt', FrozenKeys({'BLOCK_M': block_m, 'BLOCK_N': block_n}), arg_defs


def _leading_dim(x: torch.Tensor) -> int:
    """Distance in elements between consecutive k of a `[rows, k]` tensor whose rows are contiguous."""
    rows, k = x.shape
    assert rows <= 1 or x.stride(0) == 1, 'a and b must have their first dimension contiguous (get_col_major_tensor)'
    ld = x.stride(1) if k > 1 else rows
    assert ld >= rows and ld % 4 == 0
    return ld


def gemm_float_nt(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor,
                  alpha: float = 1.0, beta: float = 0.0) -> None:
    m, k = a.shape
    n, k_ = b.shape
    m_, n_ = c.shape

    assert m % 128 == 0 and n % 64 == 0

    assert m == m_ and n == n_ and k == k_
    assert a.dtype == torch.float32 and b.dtype == torch.float32 and c.dtype == torch.float32
    assert c.is_contiguous()

    if m == 0 or n == 0:
        return

    ldA, ldB, ldC = _leading_dim(a), _leading_dim(b), n
    stream = current_raw_stream()
    args = (m, n, k, float(alpha), a, ldA, b, ldB, float(beta), c, ldC, stream)
    name, keys, defs = float_kernel_plan(m, n, get_num_sms())
    runtime = jit_tuner.compile_and_tune(name=name, keys=keys, space=(), includes=includes,
                                         arg_defs=defs, template=template, args=args)
    rc = runtime(*args)
    assert rc == 0, f'{name} failed with HIP error {rc}'


def accuracy_test():
    """The reference's smoke check (`simple_gemm.py:59-73`): seed 42, 5120 x 2048 x 4096, against `a @ b.t()`."""
    from .utils import get_col_major_tensor
    torch.manual_seed(42)
    m, n, k = 5120, 2048, 4096
    a = torch.randn(m, k, dtype=torch.float32, device='cuda')
    b = torch.randn(n, k, dtype=torch.float32, device='cuda')
    c = torch.zeros(m, n, dtype=torch.float32, device='cuda')
    c_ref = a.double() @ b.double().t()
    gemm_float_nt(get_col_major_tensor(a), get_col_major_tensor(b), c)
    assert torch.allclose(c.double(), c_ref, rtol=1e-4, atol=1e-3)
    print('Simple GEMM test passed!')
