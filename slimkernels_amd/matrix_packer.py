"""Host-side 2-bit packer: the interchange layout of W2A8 weights.

Drop-in for the upstream ``matrix_packer.py`` (same function names, argument
meaning, return types, exception types and message texts; upstream
matrix_packer.py:3-36 and :38-66).  Four codes (values 0..3) share one byte;
the first code of each quadruple occupies bits 7:6 and the fourth bits 1:0
(matrix_packer.py:33-34).  This is offline weight preparation and runs on the
host in numpy, as it does upstream; the GPU consumes its output through
``slimkernels_amd.torch.repack_w2``.
"""
import numpy as np

_SHIFTS = np.array([6, 4, 2, 0], dtype=np.uint8)


def pack_matrix(input_matrix):
    """uint8 [R, C] holding 2-bit codes -> uint8 [R, C/4].

    Raises ValueError with the upstream message texts (matrix_packer.py:14,17,21)
    for a non-uint8 dtype, a column count that is not a multiple of four, or a
    value outside 0..3.
    """
    if input_matrix.dtype != np.uint8:
        raise ValueError("输入矩阵必须是uint8类型")
    if input_matrix.shape[1] % 4 != 0:
        raise ValueError("输入矩阵的列数必须是4的倍数")
    if input_matrix.size and int(input_matrix.max()) > 3:
        raise ValueError("输入矩阵的值必须在0-3之间")
    quads = input_matrix.reshape(input_matrix.shape[0], input_matrix.shape[1] // 4, 4)
    return np.bitwise_or.reduce(quads << _SHIFTS, axis=2).astype(np.uint8)


def unpack_matrix(packed_matrix):
    """Inverse of :func:`pack_matrix` (matrix_packer.py:57-64): uint8 [R, P] -> uint8 [R, 4P]."""
    if packed_matrix.dtype != np.uint8:
        raise ValueError("输入矩阵必须是uint8类型")
    fields = (packed_matrix[:, :, None] >> _SHIFTS) & np.uint8(3)
    return fields.reshape(packed_matrix.shape[0], packed_matrix.shape[1] * 4).astype(np.uint8)
