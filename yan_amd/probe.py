"""Measurement helpers that are not part of the operator surface: the rate the matrix cores sustain with nothing to
fetch (`mfma_ceiling`), which is what a GEMM kernel's MFMA roofline fraction should be read against on a chip that is
power-limited under this load. Built through the same JIT as the GEMM kernels."""
import torch

from .jit import build, generate
from .jit_kernels.utils import get_num_sms

_includes = ('"probe/mfma_ceiling.hpp"', )
_arg_defs = (('mode', int), ('src', torch.int), ('out', torch.float), ('num_cus', int), ('iters', int), ('stream', torch.cuda.Stream))
_body = """
using namespace yan;
__return_code = static_cast<int>(launch_mfma_ceiling(mode, src, out, num_cus, iters, stream));
"""
MODES = {'bf16_32x32x16': 0, 'bf16_16x16x32': 1, 'fp8_16x16x128_accumulate': 2, 'fp8_16x16x128_zero_c_plus_fold': 3,
         'fp8_fold_plus_lds_reads': 4, 'fp8_fold_plus_lds_reads_barrier': 5, 'fp8_fold_plus_lds_reads_barrier_copies': 6}
_FLOPS_PER_WAVE_ITER = {0: 16 * 2 * 32 * 32 * 16, 1: 16 * 2 * 16 * 16 * 32, **{mode: 32 * 2 * 16 * 16 * 128 for mode in range(2, 7)}}


def probe_kernel():
    """(name, arg_defs, code) of the probe's JIT kernel; needs no GPU."""
    return 'mfma_ceiling', _arg_defs, generate(_includes, _arg_defs, _body)


def mfma_ceiling(kind: str, data: str = 'random', iters: int = 4000, launches: int = 20) -> float:
    """TFLOPS of a register-resident MFMA loop on every CU. `data`: 'random' (operand bits of N(0,1) values: bf16
    numbers, or e4m3 codes of values scaled to the format's range) or 'zero'."""
    mode = MODES[kind]
    cus = get_num_sms()
    words = cus * 8 * 12 * 64 * 8
    if data == 'zero':
        src = torch.zeros(words, dtype=torch.int, device='cuda')
    elif mode < 2:
        src = torch.randn(words * 2, device='cuda').bfloat16().view(torch.int)
    else:
        x = torch.randn(words * 4, device='cuda')
        src = (x * (448.0 / x.abs().max())).to(torch.float8_e4m3fn).view(torch.int)
    out = torch.empty(cus * 512, dtype=torch.float, device='cuda')
    runtime = build(*probe_kernel())
    args = (mode, src, out, cus, iters, torch.cuda.current_stream())
    for _ in range(3):
        assert runtime(*args) == 0
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(launches):
        runtime(*args)
    end.record()
    end.synchronize()
    seconds = start.elapsed_time(end) * 1e-3 / launches
    waves = 4 if mode == 0 else 8
    return _FLOPS_PER_WAVE_ITER[mode] * waves * cus * iters / seconds / 1e12
