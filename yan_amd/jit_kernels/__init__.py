from .bf16_gemm import gemm_bf16_tn, gemm_fp16_tn, accuracy_test as bf16_gemm_accuracy_test
from .bf16_gemm import accuracy_test as cute_gemm_accuracy_test      # the reference's name for it (yan/jit_kernels/__init__.py:2)
from .gemm import gemm_bf16_fp8_bf16_nt, gemm_fp8_fp8_bf16_nt
from .simple_gemm import gemm_float_nt, accuracy_test as simple_gemm_accuracy_test
from .m_grouped_gemm import m_grouped_gemm_fp8_fp8_bf16_nt_contiguous, m_grouped_gemm_fp8_fp8_bf16_nt_masked
from .fp8_cast import per_token_cast_to_fp8, per_block_cast_to_fp8
from .utils import (ceil_div, set_num_sms, get_num_sms, get_col_major_tensor, get_m_alignment_for_contiguous_layout,
                    compare_tensors)
from .tuner import jit_tuner
