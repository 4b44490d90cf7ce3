"""The FP8 GEMM entry point that allocates nothing (yan_gemm_fp8_fp8_bf16_nt_static): split-K on the library's own device
array instead of a caller's workspace. Checked against the workspace entry point through the C ABI."""
import pytest
import torch

import harness as testing
from yan_amd import capi

pytestmark = pytest.mark.gpu


def test_static_scratch_entry_point_matches_the_workspace_entry_point():
    """Two calls in a row on one array, the second on a smaller problem with another tile and factor, then a problem whose K
    is not split: the bits of the workspace entry point every time, nothing written past the output, and the device's free
    memory unchanged over a second round (the first loads the kernels)."""
    assert torch.cuda.is_available(), 'this test needs a GPU'
    torch.cuda.set_device(0)
    shapes = [(256, 7168, 7168), (33, 2112, 5376), (300, 96, 640)]
    assert capi.select_split_k(*shapes[0], 256) == (128, 128, 2) and capi.select_split_k(*shapes[1], 256) == (64, 32, 3)
    assert capi.select_split_k(*shapes[2], 256) is None
    workspace = capi.split_k_workspace()
    cases = [testing.make_fp8_case(*shape, seed=31 + i, device='cuda', gen_device='cuda') for i, shape in enumerate(shapes)]
    expected = []
    for (lhs, rhs, out) in cases:
        assert capi.gemm_fp8_fp8_bf16_nt_split_k(lhs, rhs, out, workspace) == 0
        expected.append(out.clone())
    torch.cuda.synchronize()
    for ((a8, sa), (b8, sb), _), want in zip(cases, expected):
        ref = testing.dequant_lhs(a8, sa) @ testing.dequant_rhs(b8, sb).t()
        num, den = 2 * (want.double() * ref.double()).sum(), (want.double() ** 2 + ref.double() ** 2).sum()
        assert float(1 - num / den) < 1e-5
    free_before = None
    for round_ in range(2):
        for (shape, (lhs, rhs, _), want) in zip(shapes, cases, expected):
            print('[case] static scratch', shape, 'round', round_, flush=True)
            m, n = shape[0], shape[1]
            padded = torch.full((m + 2, n), 7.0, dtype=torch.bfloat16, device='cuda')
            assert capi.gemm_fp8_fp8_bf16_nt_static(lhs, rhs, padded) == 0
            torch.cuda.synchronize()
            assert torch.equal(padded[:m], want) and bool((padded[m:] == 7.0).all())
            del padded
        free_now = torch.cuda.mem_get_info()[0]
        if free_before is not None:
            assert free_now == free_before
        free_before = free_now


def test_reset_clears_the_arrival_counters_of_a_workspace():
    """yan_gemm_split_k_reset: counters that something left dirty (here: written by hand) are zero again after the call,
    for a caller's workspace and, with a null workspace, for the library's own array; the next split-K call on either
    gives the bits of a clean run, and the reset itself allocates nothing."""
    torch.cuda.set_device(0)
    lib = capi.load()
    counter_bytes = lib.yan_gemm_split_k_counter_bytes()
    lhs, rhs, out = testing.make_fp8_case(64, 4096, 7168, seed=41, device='cuda', gen_device='cuda')
    assert capi.select_split_k(64, 4096, 7168, 256) is not None
    workspace = capi.split_k_workspace()
    assert capi.gemm_fp8_fp8_bf16_nt_split_k(lhs, rhs, out, workspace) == 0
    torch.cuda.synchronize()
    want = out.clone()
    assert int(workspace[:counter_bytes].max()) == 0
    print('[case] reset of a dirty workspace', flush=True)
    workspace[:counter_bytes].fill_(1)
    free_before = torch.cuda.mem_get_info()[0]
    assert capi.split_k_reset(workspace) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert int(workspace[:counter_bytes].max()) == 0
    assert int(workspace[counter_bytes:counter_bytes + 4096].max()) > 0         # partial sums are left alone
    out.zero_()
    assert capi.gemm_fp8_fp8_bf16_nt_split_k(lhs, rhs, out, workspace) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    print('[case] reset of the static array', flush=True)
    assert capi.split_k_reset(None) == 0
    out.zero_()
    assert capi.gemm_fp8_fp8_bf16_nt_static(lhs, rhs, out) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, want)
