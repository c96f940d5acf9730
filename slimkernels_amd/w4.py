"""4-bit weights for the W2A8 kernels: a W4 matrix is two 2-bit planes.

Upstream only sketches W4 (slimkernels/triton/gemm_splitk.ipynb cell 0: ``w4matmul_splitk`` on random
packed integers, eight 4-bit codes per uint32 along K, code k % 8 at bits 4 * (k % 8), fp16 activations,
no scales); it has no W4 quantiser and no tests, so the quantiser below is this build's own, shaped like
its W2 one.  The arithmetic needs no new kernel: a 4-bit code c = 4 * hi + lo with hi, lo in 0..3, so

    sum_k q[k] * (c[k] - zp4) = 4 * sum_k q[k] * (hi[k] - (zp4 >> 2)) + sum_k q[k] * (lo[k] - (zp4 & 3))

and a W4 GEMM over K with G scale groups is a W2 GEMM over 2K with 2G groups: the hi plane first, with
scales 4 * s and zero-points zp4 >> 2, then the lo plane with scales s and zero-points zp4 & 3, against the
activation row written twice.  Weight bytes are those of a native 4-bit layout (two 2-bit planes of K/4
bytes per row); the matrix cores do twice the work of a native 4-bit unpack, which costs nothing where the
weight stream bounds the time (few token rows) and half the rate where the matrix cores do (prefill).
"""
import numpy as np

from .matrix_packer import pack_matrix
from .quantization import _check_groups

_QMAX4 = 15


def pack_w4(codes):
    """uint8 [N, K] with values 0..15 -> uint8 [N, K/2]: two codes per byte along K, the first in the high
    nibble (the rule of pack_matrix, matrix_packer.py:33-34, at four bits)."""
    codes = np.asarray(codes)
    if codes.dtype != np.uint8:
        raise ValueError("codes must be uint8")
    if codes.ndim != 2 or codes.shape[1] % 2 != 0:
        raise ValueError("codes must be 2-D with an even number of columns")
    if codes.size and int(codes.max()) > _QMAX4:
        raise ValueError("codes must be in 0..15")
    return ((codes[:, 0::2] << 4) | codes[:, 1::2]).astype(np.uint8)


def unpack_w4(packed):
    """Inverse of pack_w4: uint8 [N, K/2] -> uint8 [N, K]."""
    packed = np.asarray(packed)
    if packed.dtype != np.uint8 or packed.ndim != 2:
        raise ValueError("packed must be a 2-D uint8 array")
    out = np.empty((packed.shape[0], packed.shape[1] * 2), dtype=np.uint8)
    out[:, 0::2] = packed >> 4
    out[:, 1::2] = packed & 0xF
    return out


def codes_from_uint32_kn(packed_b):
    """The upstream notebook's W4 operand, uint32 [K/8, N] with code k % 8 of word k // 8 at bits 4 * (k % 8)
    (gemm_splitk.ipynb cell 0: ``(b >> (offs_k % 8) * 4) & 0xF``) -> codes uint8 [N, K]."""
    b = np.asarray(packed_b)
    if b.ndim != 2:
        raise ValueError("packed_b must be 2-D [K/8, N]")
    b = b.astype(np.uint32, copy=False)
    k8, n = b.shape
    out = np.empty((k8, 8, n), dtype=np.uint8)
    for j in range(8):
        out[:, j, :] = (b >> np.uint32(4 * j)) & np.uint32(0xF)
    return np.ascontiguousarray(out.reshape(k8 * 8, n).T)


def quantize_w4(matrix, group_size=128, mode="sym"):
    """[K, N] float array -> (codes uint8 [K, N], scales float32 [G, N], zero-points uint8 [G, N]); groups
    of ``group_size`` rows, one scale per group and column, fp32 arithmetic, ties to even.
    "sym": levels -8..7, s = max(absmax, 1e-9) / 8, zero-point 8.
    "asym": s = max(max - min, 1e-9) / 15, zp = clip(rne(-min / s), 0, 15)."""
    if not isinstance(matrix, np.ndarray):
        raise TypeError("Input must be a numpy array")
    num_rows, num_cols = matrix.shape
    num_groups = _check_groups(num_rows, group_size)
    grouped = matrix.astype(np.float32, copy=False).reshape(num_groups, group_size, num_cols)
    tiny = np.float32(1e-9)
    if mode == "sym":
        scales = np.maximum(np.abs(grouped).max(axis=1, keepdims=True), tiny) / np.float32(8.0)
        zero = np.full_like(scales, 8)
    elif mode == "asym":
        low = grouped.min(axis=1, keepdims=True)
        scales = np.maximum(grouped.max(axis=1, keepdims=True) - low, tiny) / np.float32(15.0)
        zero = np.clip(np.round(-low / scales), 0, _QMAX4).astype(np.float32)
    else:
        raise ValueError(f"unknown quantizer mode {mode!r} (expected 'sym' or 'asym')")
    scales = scales.astype(np.float32)
    levels = grouped / scales
    np.round(levels, out=levels)
    levels += zero
    np.clip(levels, 0, _QMAX4, out=levels)
    return (levels.astype(np.uint8).reshape(num_rows, num_cols), scales.reshape(num_groups, num_cols),
            zero.reshape(num_groups, num_cols).astype(np.uint8))


def prepare_w4(weight_nk, group_size=128, mode="sym"):
    """fp weight [N, K] (the nn.Linear orientation) -> (packed uint8 [N, K/2], scales float16 [G, N],
    zero-points uint8 [G, N]); groups run along K."""
    w = np.asarray(weight_nk)
    codes, scales, zero = quantize_w4(np.ascontiguousarray(w.T), group_size, mode)
    return pack_w4(np.ascontiguousarray(codes.T)), scales.astype(np.float16), zero


def split_planes(codes_nk, scales, zp):
    """4-bit codes [N, K], scales float16 [G, N], zero-points uint8 [G, N] (values 0..15) -> the W2 operand
    over 2K: (packed uint8 [N, 2K/4] in the pack_matrix byte order, scales float16 [2G, N], zero-points
    uint8 [2G, N] with values 0..3).  Columns 0..K-1 are the hi plane (codes >> 2, scales 4 * s, zero-points
    zp >> 2), columns K..2K-1 the lo plane (codes & 3, scales s, zero-points zp & 3)."""
    codes_nk = np.asarray(codes_nk)
    scales = np.asarray(scales)
    zp = np.asarray(zp)
    if codes_nk.dtype != np.uint8 or codes_nk.ndim != 2:
        raise ValueError("codes must be a 2-D uint8 array [N, K]")
    if scales.dtype != np.float16 or zp.dtype != np.uint8 or scales.shape != zp.shape:
        raise ValueError("scales must be float16 and zero-points uint8, both [G, N]")
    if codes_nk.size and int(codes_nk.max()) > _QMAX4 or zp.size and int(zp.max()) > _QMAX4:
        raise ValueError("codes and zero-points must be in 0..15")
    with np.errstate(over="ignore"):
        hi_scale = (scales.astype(np.float32) * np.float32(4.0)).astype(np.float16)
    if not np.all(np.isfinite(hi_scale)):
        raise ValueError("4 * scale overflows float16")
    planes = np.concatenate([codes_nk >> 2, codes_nk & 3], axis=1)
    return (pack_matrix(planes), np.concatenate([hi_scale, scales], axis=0),
            np.concatenate([zp >> 2, zp & 3], axis=0).astype(np.uint8))
