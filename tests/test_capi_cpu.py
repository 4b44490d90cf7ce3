"""The ahead-of-time C-ABI library without a GPU: it loads, exports exactly what include/yan_gemm.h declares, its
host-only entry points work, and its compute entry points reject bad sizes before any device call."""
import ctypes
import os
import re
import subprocess

import pytest

import yan_amd as yan
from yan_amd import capi
from yan_amd.jit_kernels import heuristics


@pytest.fixture(scope='module')
def lib():
    return capi.load()


def _declared(repo_root):
    text = open(os.path.join(repo_root, 'include', 'yan_gemm.h')).read()
    return sorted(re.findall(r'^YAN_API\s+[\w\s\*]+?\b(yan_\w+)\s*\(', text, flags=re.M))


def test_library_exports_every_declared_symbol(lib, repo_root):
    declared = _declared(repo_root)
    assert declared == sorted(capi.SYMBOLS) and len(declared) == 18
    for name in declared:
        assert hasattr(lib, name), name
    out = subprocess.check_output(['nm', '-D', '--defined-only', os.path.join(repo_root, 'yan_amd', 'csrc', 'libyan_gemm.so')], text=True)
    exported = sorted(ln.split()[-1] for ln in out.splitlines() if ' T ' in ln)
    assert exported == declared          # nothing else leaks out of the library


def test_header_is_plain_c(repo_root, tmp_path):
    src = tmp_path / 'use.c'
    src.write_text('#include "yan_gemm.h"\nconst char* (*probe)(void) = yan_gemm_version;\nint main(void) { yan_jit_launch_dense_fn f = 0; yan_jit_launch_fp8_fn g = 0; (void)f; (void)g; return probe ? 0 : 1; }\n')
    subprocess.check_call(['gcc', '-std=c99', '-Wall', '-Werror', '-pedantic', '-c', str(src), '-I', os.path.join(repo_root, 'include'),
                           '-o', str(tmp_path / 'use.o')])


def test_version_and_tile_selection_match_python(lib):
    assert b'gfx950' in lib.yan_gemm_version()
    shapes = [(4096, 7168, 7168), (64, 4096, 7168), (16384, 16384, 16384), (8192, 8192, 8192), (1024, 1024, 1024),
              (1, 128, 128), (300, 96, 640), (1, 4096, 7168), (17, 4096, 1024), (33, 2112, 640), (64, 7168, 2048), (65, 7168, 2048), (257, 2112, 1024), (256, 24576, 1536), (4096, 2048, 7168), (129, 320, 128)]
    for m, n, k in shapes:
        for cus in (256, 128, 80):
            assert capi.select_tile(0, m, n, k, cus) == heuristics.get_dense_tile(m, n, k, cus), (m, n, k, cus)
            assert capi.select_tile(1, m, n, k, cus) == heuristics.get_fp8_tile(m, n, k, cus), (m, n, k, cus)
    picked_on_device = 0
    for m, n in [(4096, 4096), (32768, 4096), (128, 7168), (256, 200), (1024, 24576), (8192, 4096), (8192, 7168), (6144, 2112), (16384, 4096)]:
        for cus in (256, 80):
            for groups in (1, 4, 8, 16, 64):
                assert capi.select_tile(2, m, n, groups, cus) == heuristics.get_best_grouped_fp8_config(m, n, 1024, cus, 1, 128, groups)
                assert capi.select_tile(4, m, n, groups, cus) == ((256, 256) if heuristics.get_contiguous_rows_on_device(m, n, 1024, cus, groups) else (0, 0))
                picked_on_device += heuristics.get_contiguous_rows_on_device(m, n, 1024, cus, groups)
    assert picked_on_device >= 6
    for m, n in [(128, 2112), (128, 24576), (128, 32768), (128, 7168), (4096, 7168), (4096, 2112), (4096, 32768), (128, 64), (5120, 2048),
                 (256, 256), (512, 4096), (1024, 1024), (2048, 2048), (256, 32768)]:
        for cus in (256, 80):
            assert capi.select_tile(3, m, n, 512, cus) == heuristics.get_best_float_config(m, n, cus), (m, n, cus)
    # the split-K plan of the plain FP8 GEMM: same rule, same numbers on both sides
    plans = 0
    for m in (1, 16, 17, 32, 33, 50, 64, 65, 100, 128, 129, 200, 256, 300, 512, 700, 1024, 4096):
        for n in (100, 196, 516, 1536, 2112, 4096, 4100, 7168, 16384, 24576):
            for k in (128, 1536, 2048, 3072, 3200, 4608, 6144, 7168, 16384):
                for cus in (256, 64, 40, 8):
                    plan = capi.select_split_k(m, n, k, cus)
                    assert plan == heuristics.get_split_k_fp8_config(m, n, k, cus), (m, n, k, cus)
                    dense_plan = capi.select_split_k(m, n, k, cus, op=0)
                    assert dense_plan == heuristics.get_split_k_dense_config(m, n, k, cus), (m, n, k, cus)
                    plans += (plan is not None) + (dense_plan is not None)
    assert plans > 1000
    assert lib.yan_gemm_split_k_workspace_bytes() == yan.gemm.SPLIT_K_WORKSPACE_BYTES == 16 * 1024 + 256 * 128 * 128 * 4
    assert lib.yan_gemm_split_k_counter_bytes() == yan.gemm.SPLIT_K_COUNTER_BYTES
    bm, bn = ctypes.c_int(), ctypes.c_int()
    assert lib.yan_gemm_select_split_k(1, 64, 4096, 7168, 0, ctypes.byref(bm), ctypes.byref(bn), ctypes.byref(bm)) == 1
    assert lib.yan_gemm_select_split_k(2, 64, 4096, 7168, 256, ctypes.byref(bm), ctypes.byref(bn), ctypes.byref(bm)) == 1
    assert lib.yan_gemm_select_tile(7, 1, 1, 1, 256, ctypes.byref(bm), ctypes.byref(bn)) == 1
    assert lib.yan_gemm_select_tile(0, 1, 1, 1, 0, ctypes.byref(bm), ctypes.byref(bn)) == 1


def test_compute_entry_points_validate_before_touching_a_device(lib):
    null = ctypes.c_void_p(0)
    assert lib.yan_gemm_bf16_tn(0, 64, 64, null, null, null, null) == 0          # empty problem: no-op
    assert lib.yan_gemm_fp16_tn(64, 0, 64, null, null, null, null) == 0
    assert lib.yan_gemm_bf16_tn(-1, 64, 64, null, null, null, null) != 0
    assert lib.yan_gemm_bf16_tn(64, 62, 64, null, null, null, null) != 0         # n % 4
    assert lib.yan_gemm_bf16_tn(64, 64, 60, null, null, null, null) != 0         # k % 8
    assert lib.yan_gemm_bf16_tn(64, 64, 64, null, null, null, null) != 0         # null operands
    f = ctypes.c_float
    assert lib.yan_gemm_float_nt(0, 64, 16, f(1), null, 0, null, 64, f(0), null, 64, null) == 0            # empty problem
    assert lib.yan_gemm_float_nt(128, 64, 16, f(1), null, 128, null, 64, f(0), null, 64, null) != 0        # null operands
    aligned = ctypes.c_void_p(4096)
    assert lib.yan_gemm_float_nt(126, 64, 16, f(1), aligned, 128, aligned, 64, f(0), aligned, 64, null) != 0   # m % 4
    assert lib.yan_gemm_float_nt(128, 64, 16, f(1), aligned, 64, aligned, 64, f(0), aligned, 64, null) != 0    # lda < m
    assert lib.yan_gemm_float_nt(128, 64, 16, f(1), aligned, 128, aligned, 64, f(0), aligned, 60, null) != 0   # ldc < n
    assert lib.yan_gemm_float_nt(128, 64, 16, f(1), ctypes.c_void_p(4100), 128, aligned, 64, f(0), aligned, 64, null) != 0   # alignment
    assert lib.yan_gemm_float_nt(128, 64, 1 << 22, f(1), aligned, 128, aligned, 64, f(0), aligned, 64, null) != 0   # beyond 32-bit offsets
    assert lib.yan_gemm_fp8_fp8_bf16_nt(null, null, 1, 1, null, null, null, 0, 128, 128, null, 256) == 0
    assert lib.yan_gemm_fp8_fp8_bf16_nt(null, null, 1, 1, null, null, null, 4, 128, 64, null, 256) != 0    # k % 128
    assert lib.yan_gemm_fp8_fp8_bf16_nt(null, null, 1, 1, null, null, null, 4, 126, 128, null, 256) != 0   # n % 4
    assert lib.yan_gemm_fp8_fp8_bf16_nt(null, null, 1, 1, null, null, null, 4, 128, 128, null, 256) != 0   # null operands
    assert lib.yan_per_token_cast_to_fp8(null, 0, null, null, 1, 1, 0, 128, null) == 0                     # no rows
    assert lib.yan_per_token_cast_to_fp8(null, 0, null, null, 1, 1, 4, 100, null) != 0                     # k % 128
    assert lib.yan_per_token_cast_to_fp8(null, 1, null, null, 1, 1, 4, 128, null) != 0                     # null operands
    assert lib.yan_per_block_cast_to_fp8(null, 0, null, null, 0, 128, null) == 0
    assert lib.yan_per_block_cast_to_fp8(null, 1, null, null, 4, 130, null) != 0
    assert lib.yan_per_block_cast_to_fp8(null, 0, null, null, 4, 128, null) != 0
    grouped_c, grouped_m = lib.yan_m_grouped_gemm_fp8_fp8_bf16_nt_contiguous, lib.yan_m_grouped_gemm_fp8_fp8_bf16_nt_masked
    assert grouped_c(null, null, 1, 1, null, null, null, null, 2, 0, 128, 128, null, 256) == 0             # no rows
    assert grouped_c(null, null, 1, 1, null, null, null, null, 2, 100, 128, 128, null, 256) != 0           # m % 128
    assert grouped_c(null, null, 1, 1, null, null, null, null, 2, 128, 128, 64, null, 256) != 0            # k % 128
    assert grouped_c(null, null, 1, 1, null, null, null, null, 0, 128, 128, 128, null, 256) != 0           # no groups
    assert grouped_c(null, null, 1, 1, null, null, null, null, 2, 128, 128, 128, null, 256) != 0           # null operands
    assert grouped_m(null, null, 1, 1, 1, null, null, null, null, 0, 64, 64, 128, 128, null, 256) == 0     # no groups
    assert grouped_m(null, null, 1, 1, 1, null, null, null, null, 2, 64, 0, 128, 128, null, 256) != 0      # expected_m
    assert grouped_m(null, null, 1, 1, 1, null, null, null, null, 2, 64, 64, 126, 128, null, 256) != 0     # n % 4
    assert grouped_m(null, null, 1, 1, 1, null, null, null, null, 2, 64, 64, 128, 128, null, 256) != 0     # null operands
