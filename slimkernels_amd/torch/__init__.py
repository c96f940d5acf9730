"""PyTorch-ROCm entry points of the W2A8 GEMM path (torch is used for device memory
and streams only; all arithmetic runs in the HIP kernels behind the C ABI)."""
from .convert import replace_linears
from .w4 import W4A8Linear, W4A8Weight, load_w4_weight, quantize_weight4_gpu, repack_w4, save_w4, w4a8_gemm, w4a8_gemm_grouped, w4a8_linear, w4matmul_splitk
from .ops import (W2A16Linear, W2A8Linear, W2A8Weight, fused_applies, load_w2_weight, needs_rowsum, quantize_act_int8, quantize_weight_gpu, repack_w2, w2a16_gemm, w2a16_gemm_grouped, w2a8_gemm, w2a8_gemm_grouped,
                  w2a8_linear_fused, wint2_gemm)

__all__ = ["W2A16Linear", "W2A8Linear", "W2A8Weight", "W4A8Linear", "W4A8Weight", "load_w4_weight", "quantize_weight4_gpu", "repack_w4", "save_w4", "w4a8_gemm_grouped", "w4a8_gemm", "w4a8_linear", "w4matmul_splitk", "fused_applies", "load_w2_weight", "needs_rowsum", "quantize_act_int8", "quantize_weight_gpu", "repack_w2", "replace_linears", "w2a16_gemm", "w2a16_gemm_grouped", "w2a8_gemm", "w2a8_gemm_grouped",
           "w2a8_linear_fused", "wint2_gemm"]
