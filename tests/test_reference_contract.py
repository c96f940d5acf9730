"""The upstream repository's own pytest cases (test_matrix_packer.py, test_quantization.py),
re-expressed against slimkernels_amd's host-side drop-ins: same inputs, same expected
arrays, same exception types and message patterns."""
import numpy as np
import pytest

from slimkernels_amd import (dequantize_from_uint2, pack_matrix, quantize_to_uint2, unpack_matrix)

CODES_4x8 = np.array([[0, 1, 2, 3, 0, 1, 2, 3],
                      [3, 2, 1, 0, 3, 2, 1, 0],
                      [1, 1, 1, 1, 2, 2, 2, 2],
                      [0, 3, 2, 1, 3, 0, 1, 2]], dtype=np.uint8)
PACKED_4x2 = np.array([[27, 27], [228, 228], [85, 170], [57, 198]], dtype=np.uint8)


# ---- upstream test_matrix_packer.py
def test_pack_known_answer():  # :5-25
    np.testing.assert_array_equal(pack_matrix(CODES_4x8), PACKED_4x2)


def test_pack_invalid_input():  # :27-41
    with pytest.raises(ValueError, match="输入矩阵的值必须在0-3之间"):
        pack_matrix(np.array([[0, 1, 2, 4]], dtype=np.uint8))
    with pytest.raises(ValueError, match="输入矩阵的列数必须是4的倍数"):
        pack_matrix(np.array([[0, 1, 2]], dtype=np.uint8))
    with pytest.raises(ValueError, match="输入矩阵必须是uint8类型"):
        pack_matrix(np.array([[0, 1, 2, 3]], dtype=np.float32))


def test_unpack_known_answer():  # :43-61
    np.testing.assert_array_equal(unpack_matrix(PACKED_4x2), CODES_4x8)


def test_pack_unpack_roundtrip():  # :63-72
    original = np.random.default_rng(7).integers(0, 4, (10, 8), dtype=np.uint8)
    np.testing.assert_array_equal(unpack_matrix(pack_matrix(original)), original)


def test_unpack_rejects_non_uint8():  # matrix_packer.py:48-49
    with pytest.raises(ValueError, match="输入矩阵必须是uint8类型"):
        unpack_matrix(PACKED_4x2.astype(np.int32))


# ---- upstream test_quantization.py
def test_basic_quantization():  # :5-27
    matrix = np.array([[1.0, -2.0], [3.0, -4.0], [5.0, -6.0], [7.0, -8.0],
                       [9.0, -10.0], [11.0, -12.0], [13.0, -14.0], [15.0, -16.0]])
    quantized, scales = quantize_to_uint2(matrix, group_size=8)
    assert quantized.dtype == np.uint8
    assert np.all(quantized >= 0) and np.all(quantized <= 3)
    assert scales.shape == (1, 2)


def test_quantize_invalid_input():  # :29-38
    with pytest.raises(TypeError):
        quantize_to_uint2([[1, 2], [3, 4]])
    with pytest.raises(ValueError):
        quantize_to_uint2(np.random.default_rng(0).standard_normal((10, 4)), group_size=8)


def test_zero_handling():  # :40-48
    quantized, scales = quantize_to_uint2(np.zeros((8, 2)))
    assert np.all(quantized == 1)
    assert np.all(scales > 0)


def test_multiple_groups():  # :50-56
    quantized, scales = quantize_to_uint2(np.random.default_rng(1).standard_normal((16, 4)), group_size=8)
    assert scales.shape == (2, 4)
    assert quantized.shape == (16, 4)


def test_extreme_values():  # :58-75
    matrix = np.array([[1e6, -1e6], [1e-6, -1e-6], [0.0, 0.0], [1.0, -1.0],
                       [10.0, -10.0], [100.0, -100.0], [1000.0, -1000.0], [10000.0, -10000.0]])
    quantized, _ = quantize_to_uint2(matrix)
    assert np.all(quantized >= 0) and np.all(quantized <= 3)


def test_dequantize_invalid_input():  # :78-97
    quantized = np.array([[0, 1], [2, 3]], dtype=np.uint8)
    scales = np.array([[1.0, 1.0]])
    with pytest.raises(TypeError):
        dequantize_from_uint2([[0, 1], [2, 3]], scales)
    with pytest.raises(TypeError):
        dequantize_from_uint2(quantized, [[1.0, 1.0]])
    with pytest.raises(TypeError):
        dequantize_from_uint2(quantized.astype(np.float32), scales)
    with pytest.raises(ValueError):
        dequantize_from_uint2(quantized, np.array([[1.0], [1.0]]))


def test_dequantize_multiple_groups():  # :99-106
    matrix = np.random.default_rng(2).standard_normal((16, 4)).astype(np.float32)
    quantized, scales = quantize_to_uint2(matrix, group_size=8)
    deq = dequantize_from_uint2(quantized, scales, group_size=8)
    assert deq.shape == matrix.shape
    assert deq.dtype == np.float16


KAT_MATRIX = np.array([[2.0, -4.0], [1.0, -2.0], [0.5, -1.0], [-2.0, 4.0],
                       [-1.0, 2.0], [-0.5, 1.0], [0.0, 0.0], [1.5, -3.0]], dtype=np.float32)
KAT_CODES = np.array([[3, 0], [2, 0], [1, 1], [0, 3], [0, 2], [1, 1], [1, 1], [2, 0]], dtype=np.uint8)


def test_quantize_known_answer():  # :108-140
    quantized, scales = quantize_to_uint2(KAT_MATRIX, group_size=8)
    np.testing.assert_allclose(scales, np.array([[2.0 * 2 / 3, 4.0 * 2 / 3]]), rtol=1e-5)
    np.testing.assert_array_equal(quantized, KAT_CODES)


def test_quantize_keeps_input_dtype_for_scales():  # quantization.py:29-38 computes in the input dtype
    _, s32 = quantize_to_uint2(KAT_MATRIX, group_size=8)
    _, s64 = quantize_to_uint2(KAT_MATRIX.astype(np.float64), group_size=8)
    assert s32.dtype == np.float32 and s64.dtype == np.float64


def test_quantize_prints_nothing(capsys):  # the upstream debugging prints (:44-45) are not part of the contract
    quantize_to_uint2(KAT_MATRIX, group_size=8)
    assert capsys.readouterr().out == ""


def test_dequantize_known_answer():  # quantization.py:89-93: (code - 1) * scale -> float16
    quantized, scales = quantize_to_uint2(KAT_MATRIX, group_size=8)
    deq = dequantize_from_uint2(quantized, scales, group_size=8)
    expect = ((KAT_CODES.astype(np.float32) - 1) * scales).astype(np.float16)
    np.testing.assert_array_equal(deq, expect)
    # inside the clip range the reconstruction error is at most half a step
    inside = np.abs(KAT_MATRIX) <= 1.5 * scales + 1e-6
    assert np.all(np.abs(deq.astype(np.float32) - KAT_MATRIX)[inside] <= scales.repeat(8, 0)[inside] / 2 + 1e-3)
