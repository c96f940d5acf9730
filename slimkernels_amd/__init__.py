"""slimkernels_amd — MI355X (gfx950) W2A8 GEMM path.

Host-side weight preparation (numpy, mirrors the upstream module-level functions):
    pack_matrix, unpack_matrix                      (upstream matrix_packer.py)
    quantize_to_uint2, dequantize_from_uint2        (upstream quantization.py)
    quantize_w2, prepare_w2                         (parameterised level sets)
    save_w2, load_w2                                (on-disk container of the interchange layout)
    slimkernels_amd.w4: pack_w4, quantize_w4, prepare_w4, split_planes   (4-bit weights as two 2-bit planes)

GPU path (PyTorch-ROCm tensors in, HIP kernels through the C ABI in
include/slimk_w2a8.h): ``slimkernels_amd.torch`` — quantize_act_int8, repack_w2,
w2a8_gemm, wint2_gemm, W2A8Linear, replace_linears, repack_w4, w4a8_gemm, W4A8Linear.  Importing that subpackage loads
``csrc/libslimk_w2a8.so`` and raises if it is missing: there is no CPU fallback.
"""
from .matrix_packer import pack_matrix, unpack_matrix
from .packed_format import load_w2, save_w2
from .quantization import (dequantize_from_uint2, prepare_w2, quantize_to_uint2, quantize_w2)

__all__ = ["pack_matrix", "unpack_matrix", "quantize_to_uint2", "dequantize_from_uint2",
           "quantize_w2", "prepare_w2", "save_w2", "load_w2"]
__version__ = "0.1.0"
