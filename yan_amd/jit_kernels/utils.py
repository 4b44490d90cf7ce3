"""Small host helpers of the GEMM entry points (reference: `yan/jit_kernels/utils.py:6-85`).

`num_sms` keeps its name for drop-in use; on MI355X it counts compute units (256).
"""
import torch

_num_sms = None
_cu_count = None


def _device_cu_count() -> int:
    # asked once: the query costs several microseconds, as much as the host side of a whole GEMM call
    global _cu_count
    if _cu_count is None:
        _cu_count = torch.cuda.get_device_properties(device='cuda').multi_processor_count
    return _cu_count


def current_raw_stream() -> int:
    """The hipStream_t handle of the current stream of the current device as an int. `torch.cuda.current_stream()` builds
    a Stream object around it and costs 3-4 us per call, a third of the host side of a decode-shape GEMM; the JIT
    runtime takes the bare handle wherever an argument is declared a `torch.cuda.Stream`."""
    try:
        return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())
    except AttributeError:          # a torch without the raw accessor
        return torch.cuda.current_stream().cuda_stream


def set_num_sms(num_sms: int) -> None:
    """Cap the number of compute units GEMM kernels may occupy."""
    global _num_sms
    assert 0 < num_sms <= _device_cu_count()
    _num_sms = num_sms


def get_num_sms() -> int:
    """Current compute-unit cap; the device's CU count when never set."""
    global _num_sms
    if _num_sms is None:
        _num_sms = _device_cu_count()
    return _num_sms


def get_num_sms_cap() -> int:
    """The cap as the kernels' launchers take it: 0 when every compute unit may be used (never capped, or capped at the
    device's count), else the cap."""
    cap = get_num_sms()
    return 0 if cap >= _device_cu_count() else cap


def ceil_div(x: int, y: int) -> int:
    return (x + y - 1) // y


def get_m_alignment_for_contiguous_layout() -> int:
    """Row alignment of each group in an M-grouped contiguous layout: one scale block, 128 rows."""
    return 128


def get_col_major_tensor(x: torch.Tensor) -> torch.Tensor:
    """Return `x` (2-D, or 3-D batched) with the same values stored so that the second-to-last dimension is
    contiguous; `x` itself when it already is (reference: utils.py:58-85). The FP8 kernel reads activation
    scales in this layout: one K-block's scales for consecutive tokens sit next to each other."""
    assert x.dim() in (2, 3)
    batched = x if x.dim() == 3 else x.unsqueeze(0)
    rows = batched.shape[1]
    if not (batched.stride(1) == 1 and batched.stride(2) == rows):
        batched = batched.transpose(1, 2).contiguous().transpose(1, 2)
    return batched if x.dim() == 3 else batched.squeeze(0)


# From this much arithmetic on (about 40 us of kernel time) a GEMM whose activation scales are not token-contiguous gets a
# token-contiguous copy of them first: the kernels read a scale per lane and k-tile, which in the row-major layout is a
# cache line per lane (4096 x 4096 x 7168: 110 us against 96 us; 1024 x 4096 x 7168: 46.9 against 41.8), and the copy costs
# about 3 us on the device. Below it the copy costs as much as it saves (512 x 7168 x 4096: 25.8 against 24.0 us).
SCALE_RELAYOUT_MIN_FLOP = 6e10


def scales_for_kernel(scales: torch.Tensor, flop: float) -> torch.Tensor:
    """The activation scales `[m, k/128]` (or `[groups, m, k/128]`) as the FP8 kernels should be given them: as they are
    when they are token-contiguous already or the problem is small, else a token-contiguous copy (same values, so the
    same result bits; allocated from torch's caching allocator on the current stream)."""
    if flop < SCALE_RELAYOUT_MIN_FLOP or scales.size(-1) == 1 or scales.size(-2) == 1:
        return scales
    if scales.stride(-2) == 1 and scales.stride(-1) == scales.size(-2):
        return scales
    return get_col_major_tensor(scales)


def compare_tensors(actual: torch.Tensor, expected: torch.Tensor, mode: str = 'element-wise', rtol: float = 1e-5,
                    atol: float = 1e-8, diff_tolerance: float = 1e-6, verbose: bool = True) -> bool:
    """Compare a result with its expectation, print a one-line verdict and return it (reference:
    `yan/jit_kernels/utils.py:138-179`, used by its accuracy tests). `mode='element-wise'` is `torch.allclose` with
    `rtol` / `atol` and, on failure, reports the mean and the largest difference and where it sits;
    `mode='similarity'` is `calc_diff(actual, expected) <= diff_tolerance` (0 when both are all zero). A shape mismatch
    or an unknown mode fails. Passing verdicts carry their figures only when `verbose`; failures always do, and with
    `verbose` also show the first ten elements of both tensors."""
    lines = []
    if actual.shape != expected.shape:
        passed = False
        lines.append(f'Shape mismatch: {tuple(actual.shape)} vs {tuple(expected.shape)}')
    elif mode == 'element-wise':
        passed = bool(torch.allclose(actual, expected, rtol=rtol, atol=atol))
        if passed:
            lines.append(f'(Tensors are element-wise close within rtol={rtol}, atol={atol})')
        else:
            gap = (actual - expected).abs()
            worst = int(gap.argmax())
            where = [int(i) for i in torch.unravel_index(torch.tensor(worst), gap.shape)] if gap.dim() else []
            lines.append(f'Mean diff: {gap.mean().item():.6f}, Max diff: {gap.max().item():.6f}')
            lines.append(f'Max diff at {where}: {actual.flatten()[worst].item():.6f} vs {expected.flatten()[worst].item():.6f}')
    elif mode == 'similarity':
        x, y = actual.double(), expected.double()
        norm = (x * x + y * y).sum()
        diff = 0.0 if norm == 0 else float(1 - 2 * (x * y).sum() / norm)
        passed = diff <= diff_tolerance
        lines.append(f'(Difference: {diff:.6f} {"<=" if passed else ">"} Tolerance: {diff_tolerance})')
    else:
        passed = False
        lines.append(f"Invalid mode '{mode}'. Choose 'element-wise' or 'similarity'.")
    print('Verification: PASSED' if passed else 'Verification: FAILED')
    if lines and (verbose or not passed):
        print('\n'.join(lines))
    if not passed and verbose:
        print(f'Actual tensor:\n{actual.flatten()[:10]}\n')
        print(f'Expected tensor:\n{expected.flatten()[:10]}\n')
    return passed
