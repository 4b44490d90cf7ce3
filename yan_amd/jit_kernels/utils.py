"""Small host helpers of the GEMM entry points (reference: `yan/jit_kernels/utils.py:6-85`).

`num_sms` keeps its name for drop-in use; on MI355X it counts compute units (256).
"""
import torch

_num_sms = None


def _device_cu_count() -> int:
    return torch.cuda.get_device_properties(device='cuda').multi_processor_count


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
