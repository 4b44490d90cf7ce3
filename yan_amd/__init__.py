"""MI355X-native GEMM hot path behind the JIT / operator surface of zoheth/yan (`yan/__init__.py:3-5`)."""
import torch

from . import jit
from .jit_kernels import (gemm, gemm_float_nt, gemm_bf16_tn, gemm_fp16_tn, gemm_bf16_fp8_bf16_nt, gemm_fp8_fp8_bf16_nt, get_col_major_tensor,
                          m_grouped_gemm_fp8_fp8_bf16_nt_contiguous, m_grouped_gemm_fp8_fp8_bf16_nt_masked,
                          per_token_cast_to_fp8, per_block_cast_to_fp8,
                          set_num_sms, get_num_sms, ceil_div, get_m_alignment_for_contiguous_layout)
from .utils import bench_kineto, calc_diff, count_bytes
