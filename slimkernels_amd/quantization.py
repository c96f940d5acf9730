"""Host-side 2-bit group quantizer for W2A8 weights.

``quantize_to_uint2`` / ``dequantize_from_uint2`` are drop-ins for the upstream
functions of the same name (quantization.py:3-53, :55-93): the matrix is
``[K, N]``, rows are grouped ``group_size`` at a time, every (group, column)
gets one scale, codes are ``clip(round_half_even(x / s) + 1, 0, 3)`` with
``s = max(absmax, 1e-9) / 1.5`` (quantization.py:29-46), and dequantisation is
``(code - 1) * s`` cast to float16 (quantization.py:89-93).  The upstream
function also prints the whole normalised matrix twice (quantization.py:44-45);
that debugging output is not part of the contract and is not reproduced.

``quantize_w2`` is the same scheme with the level set made a parameter, which
is what the GEMM path consumes:

  mode "ref"   zero-point 1, s = absmax / 1.5           (upstream)
  mode "sym"   levels {-2,-1,0,1}, zero-point 2, s = absmax / 2
  mode "asym"  s = (max - min) / 3, per-group zero-point clip(rne(-min / s), 0, 3)

All three compute in float32 and return float32 scales; ``prepare_w2`` rounds the
scales once to float16 (the stored form) and packs the codes ``[N, K/4]``.
"""
import numpy as np

from .matrix_packer import pack_matrix

_QMAX = 3  # largest 2-bit code


def _check_groups(num_rows, group_size):
    if num_rows % group_size != 0:
        raise ValueError(
            f"Number of rows ({num_rows}) must be divisible by group_size ({group_size})")
    return num_rows // group_size


def quantize_to_uint2(matrix, group_size=8):
    """[K, N] float array -> (uint8 codes [K, N], scales [K/group_size, N] in the input dtype)."""
    if not isinstance(matrix, np.ndarray):
        raise TypeError("Input must be a numpy array")
    num_rows, num_cols = matrix.shape
    num_groups = _check_groups(num_rows, group_size)
    grouped = matrix.reshape(num_groups, group_size, num_cols)
    scales = np.maximum(np.abs(grouped).max(axis=1), 1e-9) / (_QMAX / 2)
    levels = np.round(grouped / scales[:, None, :]) + 1
    codes = np.clip(levels, 0, _QMAX).astype(np.uint8).reshape(num_rows, num_cols)
    return codes, scales


def dequantize_from_uint2(quantized, scales, group_size=8):
    """(codes [K, N], scales [K/group_size, N]) -> float16 [K, N] = (code - 1) * scale."""
    if not isinstance(quantized, np.ndarray) or not isinstance(scales, np.ndarray):
        raise TypeError("Both inputs must be numpy arrays")
    if quantized.dtype != np.uint8:
        raise TypeError("Quantized matrix must be of type uint8")
    num_rows, num_cols = quantized.shape
    num_groups = _check_groups(num_rows, group_size)
    if scales.shape != (num_groups, num_cols):
        raise ValueError(
            f"Scales shape {scales.shape} does not match expected shape {(num_groups, num_cols)}")
    centred = quantized.reshape(num_groups, group_size, num_cols).astype(np.float32) - 1
    return (centred * scales[:, None, :]).reshape(num_rows, num_cols).astype(np.float16)


def _quantize_grouped(grouped, axis, mode):
    """Quantise along ``axis`` of a float32 array whose ``axis`` spans one group.
    Returns (codes uint8, scales float32, zero-points float32), the latter two with
    ``axis`` kept as length 1."""
    tiny = np.float32(1e-9)
    if mode == "ref":
        scales = np.maximum(np.abs(grouped).max(axis=axis, keepdims=True), tiny) / np.float32(1.5)
        zero = np.ones_like(scales)
    elif mode == "sym":
        scales = np.maximum(np.abs(grouped).max(axis=axis, keepdims=True), tiny) / np.float32(2.0)
        zero = np.full_like(scales, 2)
    elif mode == "asym":
        low = grouped.min(axis=axis, keepdims=True)
        scales = np.maximum(grouped.max(axis=axis, keepdims=True) - low, tiny) / np.float32(3.0)
        zero = np.clip(np.round(-low / scales), 0, _QMAX).astype(np.float32)
    else:
        raise ValueError(f"unknown quantizer mode {mode!r} (expected 'ref', 'sym' or 'asym')")
    scales = scales.astype(np.float32)
    levels = grouped / scales
    np.round(levels, out=levels)
    levels += zero
    np.clip(levels, 0, _QMAX, out=levels)
    return levels.astype(np.uint8), scales, zero


def quantize_w2(matrix, group_size=128, mode="sym"):
    """[K, N] float array -> (codes uint8 [K, N], scales float32 [G, N], zero-points uint8 [G, N])."""
    if not isinstance(matrix, np.ndarray):
        raise TypeError("Input must be a numpy array")
    num_rows, num_cols = matrix.shape
    num_groups = _check_groups(num_rows, group_size)
    grouped = matrix.astype(np.float32, copy=False).reshape(num_groups, group_size, num_cols)
    codes, scales, zero = _quantize_grouped(grouped, 1, mode)
    return (codes.reshape(num_rows, num_cols), scales.reshape(num_groups, num_cols),
            zero.reshape(num_groups, num_cols).astype(np.uint8))


def prepare_w2(weight_nk, group_size=128, mode="sym"):
    """fp weight [N, K] (the nn.Linear orientation) -> GEMM-ready host arrays.

    Returns (packed uint8 [N, K/4], scales float16 [G, N], zero-points uint8 [G, N]).
    Groups run along K: the same numbers as quantize_w2 on the transposed matrix
    (quantization.py:26 orientation) followed by pack_matrix on the transposed codes, but
    computed in place on the [N, K] layout so that no large transpose is made."""
    w = np.asarray(weight_nk)
    num_out, num_in = w.shape
    num_groups = _check_groups(num_in, group_size)
    grouped = w.astype(np.float32, copy=False).reshape(num_out, num_groups, group_size)
    codes, scales, zero = _quantize_grouped(grouped, 2, mode)
    packed = pack_matrix(codes.reshape(num_out, num_in))
    scales_gn = np.ascontiguousarray(scales.reshape(num_out, num_groups).T).astype(np.float16)
    zero_gn = np.ascontiguousarray(zero.reshape(num_out, num_groups).T).astype(np.uint8)
    return packed, scales_gn, zero_gn
