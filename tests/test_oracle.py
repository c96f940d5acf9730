"""Pins the CPU oracle (oracle/w2a8_oracle.c + .py) before anything is compared with it.

Each oracle function is checked against something it did not produce itself: the
upstream known-answer vectors, hand-computed tables, brute-force python loops, exact
floating-point identities, or numpy/torch library routines."""
import itertools
from fractions import Fraction

import numpy as np
import pytest
import torch

from slimkernels_amd import pack_matrix, prepare_w2, quantize_w2, unpack_matrix
from test_reference_contract import CODES_4x8, KAT_CODES, KAT_MATRIX, PACKED_4x2


# ------------------------------------------------------------------ pack / unpack
def test_pack_unpack_upstream_vectors(oracle):
    for pack, unpack in ((oracle.c_pack, oracle.c_unpack), (oracle.np_pack, oracle.np_unpack)):
        np.testing.assert_array_equal(pack(CODES_4x8), PACKED_4x2)
        np.testing.assert_array_equal(unpack(PACKED_4x2), CODES_4x8)


def test_pack_exhaustive_bytes(oracle):
    """All 256 code quadruples: byte value == c0*64 + c1*16 + c2*4 + c3 (matrix_packer.py:33-34)."""
    quads = np.array(list(itertools.product(range(4), repeat=4)), dtype=np.uint8)  # [256, 4]
    expect = (quads[:, 0] * 64 + quads[:, 1] * 16 + quads[:, 2] * 4 + quads[:, 3]).astype(np.uint8)
    assert sorted(expect.tolist()) == list(range(256))
    for pack, unpack in ((oracle.c_pack, oracle.c_unpack), (oracle.np_pack, oracle.np_unpack),
                         (pack_matrix, unpack_matrix)):
        np.testing.assert_array_equal(pack(quads)[:, 0], expect)
        np.testing.assert_array_equal(unpack(expect.reshape(-1, 1)), quads)


def test_pack_error_codes(oracle):
    with pytest.raises(ValueError):
        oracle.c_pack(np.array([[0, 1, 2]], np.uint8))
    with pytest.raises(ValueError):
        oracle.c_pack(np.array([[0, 1, 2, 4]], np.uint8))


def test_pack_empty_and_ragged_rows(oracle):
    assert oracle.c_pack(np.zeros((0, 8), np.uint8)).shape == (0, 2)
    assert pack_matrix(np.zeros((0, 8), np.uint8)).shape == (0, 2)
    one = np.array([[3, 0, 0, 0]], np.uint8)
    assert oracle.c_pack(one)[0, 0] == 192 and pack_matrix(one)[0, 0] == 192


# ------------------------------------------------------------------ weight quantizer
def test_quantize_ref_upstream_vector(oracle):
    for fn in (oracle.c_quantize_w2, oracle.np_quantize_w2, quantize_w2):
        codes, scales, zp = fn(KAT_MATRIX, 8, "ref")
        np.testing.assert_array_equal(codes, KAT_CODES)
        np.testing.assert_allclose(scales, [[4 / 3, 8 / 3]], rtol=1e-6)
        assert (zp == 1).all()


def test_quantize_ref_zero_and_extreme(oracle):
    for fn in (oracle.c_quantize_w2, oracle.np_quantize_w2, quantize_w2):
        codes, scales, _ = fn(np.zeros((8, 2), np.float32), 8, "ref")
        assert (codes == 1).all() and (scales > 0).all()
        m = np.array([[1e6, -1e6], [1e-6, -1e-6], [0, 0], [1, -1], [10, -10], [100, -100],
                      [1000, -1000], [10000, -10000]], np.float32)
        codes, _, _ = fn(m, 8, "ref")
        np.testing.assert_array_equal(codes[:, 0], [3, 1, 1, 1, 1, 1, 1, 1])
        np.testing.assert_array_equal(codes[:, 1], [0, 1, 1, 1, 1, 1, 1, 1])


def test_quantize_sym_hand_table(oracle):
    """absmax 2 -> s = 1; levels clip(rne(w), -2, 1); code = level + 2.  Ties go to even."""
    w = np.array([-2.0, -1.5, -1.2, -0.5, 0.5, 0.7, 1.5, 2.0], np.float32).reshape(8, 1)
    expect = np.array([0, 0, 1, 2, 2, 3, 3, 3], np.uint8).reshape(8, 1)  # -1.5->-2, -0.5->-0, 0.5->0, 1.5->2->clip 1
    for fn in (oracle.c_quantize_w2, oracle.np_quantize_w2, quantize_w2):
        codes, scales, zp = fn(w, 8, "sym")
        np.testing.assert_array_equal(codes, expect)
        assert scales[0, 0] == 1.0 and zp[0, 0] == 2
    w2 = np.array([4.0, 2.5, -2.5, 0.0, 0.0, 0.0, 0.0, -3.0], np.float32).reshape(8, 1)  # s = 2
    expect2 = np.array([3, 3, 1, 2, 2, 2, 2, 0], np.uint8).reshape(8, 1)  # 1.25->1, -1.25->-1, -1.5->-2
    for fn in (oracle.c_quantize_w2, oracle.np_quantize_w2, quantize_w2):
        np.testing.assert_array_equal(fn(w2, 8, "sym")[0], expect2)


def test_quantize_asym_hand_table(oracle):
    """min -1, max 2 -> s = 1, zp = rne(1) = 1; code = clip(rne(w) + 1, 0, 3)."""
    w = np.array([-1.0, 0.0, 1.0, 2.0, 0.5, 1.5, -0.5, 0.2], np.float32).reshape(8, 1)
    expect = np.array([0, 1, 2, 3, 1, 3, 1, 1], np.uint8).reshape(8, 1)
    for fn in (oracle.c_quantize_w2, oracle.np_quantize_w2, quantize_w2):
        codes, scales, zp = fn(w, 8, "asym")
        np.testing.assert_array_equal(codes, expect)
        assert scales[0, 0] == 1.0 and zp[0, 0] == 1
    # all-positive group: min 1, max 4 -> s = 1, zp = clip(rne(-1), 0, 3) = 0
    wpos = np.array([1.0, 2.0, 3.0, 4.0, 1.0, 1.0, 1.0, 1.0], np.float32).reshape(8, 1)
    for fn in (oracle.c_quantize_w2, oracle.np_quantize_w2, quantize_w2):
        codes, _, zp = fn(wpos, 8, "asym")
        assert zp[0, 0] == 0
        np.testing.assert_array_equal(codes[:, 0], [1, 2, 3, 3, 1, 1, 1, 1])


@pytest.mark.parametrize("mode", ["ref", "sym", "asym"])
def test_quantize_c_numpy_product_agree(oracle, mode):
    rng = np.random.default_rng(11)
    w = (rng.standard_normal((256, 24)) * 0.02).astype(np.float16).astype(np.float32)
    a = oracle.c_quantize_w2(w, 64, mode)
    b = oracle.np_quantize_w2(w, 64, mode)
    c = quantize_w2(w, 64, mode)
    for x, y, z in zip(a, b, c):
        np.testing.assert_array_equal(x, y)
        np.testing.assert_array_equal(x, z)
    # reconstruction: inside the representable range the error is at most half a step
    codes, scales, zp = a
    deq = (codes.astype(np.float32).reshape(4, 64, 24) - zp[:, None, :]) * scales[:, None, :]
    lo, hi = (0 - zp.astype(np.float32)) * scales, (3 - zp.astype(np.float32)) * scales
    wr = w.reshape(4, 64, 24)
    inside = (wr >= lo[:, None, :]) & (wr <= hi[:, None, :])
    assert inside.mean() > 0.5
    assert np.all(np.abs(deq - wr)[inside] <= (scales[:, None, :] * 0.5000001).repeat(64, 1)[inside])
    # the dequantizer is the closed form (code - zp) * s rounded to float16
    d16 = oracle.c_dequantize_w2(codes, scales, zp, 64)
    np.testing.assert_array_equal(d16, deq.reshape(256, 24).astype(np.float16))


def test_prepare_w2_matches_transposed_quantizer(oracle):
    rng = np.random.default_rng(12)
    w_nk = (rng.standard_normal((40, 256)) * 0.02).astype(np.float32)
    for mode in ("sym", "asym", "ref"):
        packed, s16, zp = prepare_w2(w_nk, 128, mode)
        codes, s, z = oracle.c_quantize_w2(np.ascontiguousarray(w_nk.T), 128, mode)
        np.testing.assert_array_equal(packed, oracle.c_pack(np.ascontiguousarray(codes.T)))
        np.testing.assert_array_equal(s16, s.astype(np.float16))
        np.testing.assert_array_equal(zp, z)


# ------------------------------------------------------------------ half / bf16 casts of the C oracle
def test_half_and_bf16_casts(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(3)
    vals = np.concatenate([
        rng.standard_normal(2000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 2000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 5.96e-8, 2.98e-8, 2.9802322e-08,
                  2.99e-8, 6.1e-5, 6.0e-5, 1.0009766, 1.00048828125, 1.0014648], np.float32)])
    got_h = np.array([L.w2o_float_to_half(float(v)) for v in vals], np.uint16)
    np.testing.assert_array_equal(got_h, vals.astype(np.float16).view(np.uint16))
    all_h = np.arange(0, 0x7c00, 7, dtype=np.uint16)
    back = np.array([L.w2o_half_to_float(int(h)) for h in all_h], np.float32)
    np.testing.assert_array_equal(back, all_h.view(np.float16).astype(np.float32))
    got_b = np.array([L.w2o_float_to_bf16(float(v)) for v in vals], np.uint16)
    want_b = torch.from_numpy(vals).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(got_b, want_b)
    np.testing.assert_array_equal(oracle.f32_to_bf16_bits(vals), want_b)


# ------------------------------------------------------------------ activation quantizer
def test_act_quant_hand_row(oracle):
    """absmax 127 -> s_a = 1 exactly; q = rne(x): ties to even."""
    row = np.zeros(64, np.float16)
    row[:8] = [127.0, -63.5, 0.5, 1.5, 2.5, -2.5, -126.5, 100.25]
    expect = np.zeros(64, np.int8)
    expect[:8] = [127, -64, 0, 2, 2, -2, -126, 100]
    for fn in (lambda x: oracle.c_act_quant(x, 64), lambda x: oracle.np_act_quant(x, 64)):
        q, s_a, rs = fn(row.reshape(1, 64))
        assert s_a[0] == np.float32(1.0)
        np.testing.assert_array_equal(q[0], expect)
        assert rs.shape == (1, 1) and rs[0, 0] == int(expect.astype(np.int32).sum())


def test_act_quant_zero_row_and_invariants(oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((6, 256)).astype(np.float16)
    x[2] = 0
    x[4, 17] = 300.0  # outlier
    q, s_a, rs = oracle.c_act_quant(x, 64)
    q2, s2, rs2 = oracle.np_act_quant(x, 64)
    np.testing.assert_array_equal(q, q2)
    np.testing.assert_array_equal(s_a, s2)
    np.testing.assert_array_equal(rs, rs2)
    assert (q[2] == 0).all() and s_a[2] == np.float32(1e-9) / np.float32(127)
    assert np.abs(q.astype(np.int32)).max() <= 127
    am = np.abs(x.astype(np.float32)).argmax(axis=1)
    for m in (0, 1, 3, 4, 5):
        assert abs(int(q[m, am[m]])) == 127
        assert s_a[m] == np.float32(np.abs(x[m].astype(np.float32)).max()) / np.float32(127)
    np.testing.assert_array_equal(rs.T, q.astype(np.int32).reshape(6, 4, 64).sum(axis=2))


def test_act_quant_brute_force_python(oracle):
    """Scalar python restatement with numpy float32 scalars (IEEE binary32 divide, rint)."""
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((2, 64)) * 3).astype(np.float16)
    q, s_a, _ = oracle.c_act_quant(x, 64)
    for m in range(2):
        amax = np.float32(0)
        for v in x[m]:
            amax = max(amax, abs(np.float32(v)))
        s = np.float32(max(amax, np.float32(1e-9))) / np.float32(127)
        assert s == s_a[m]
        for k in range(64):
            r = np.rint(np.float32(x[m, k]) / s)
            assert int(min(max(r, -127), 127)) == int(q[m, k])


def test_act_quant_bf16_input(oracle):
    rng = np.random.default_rng(8)
    xf = rng.standard_normal((3, 128)).astype(np.float32)
    bits = oracle.f32_to_bf16_bits(xf)
    q, s_a, _ = oracle.c_act_quant(bits, 64, is_bf16=True)
    q2, s2, _ = oracle.np_act_quant(oracle.bf16_bits_to_f32(bits), 64)
    np.testing.assert_array_equal(q, q2)
    np.testing.assert_array_equal(s_a, s2)


# ------------------------------------------------------------------ int32 accumulators
def test_gemm_acc_brute_force(oracle):
    rng = np.random.default_rng(21)
    M, N, K, g = 3, 5, 32, 8
    q = rng.integers(-127, 128, (M, K), dtype=np.int8)
    codes = rng.integers(0, 4, (N, K), dtype=np.uint8)
    zp = rng.integers(0, 4, (K // g, N), dtype=np.uint8)
    acc = oracle.c_gemm_acc(q, oracle.c_pack(codes), zp, g)
    for m in range(M):
        for n in range(N):
            for gi in range(K // g):
                s = 0
                for k in range(gi * g, (gi + 1) * g):
                    s += int(q[m, k]) * (int(codes[n, k]) - int(zp[gi, n]))
                assert acc[m, n, gi] == s


@pytest.mark.parametrize("g", [64, 128])
def test_gemm_acc_exact_blas_and_zp_folding(oracle, g):
    rng = np.random.default_rng(22)
    M, N, K = 9, 70, 512
    q = rng.integers(-127, 128, (M, K), dtype=np.int8)
    q[0] = 127  # worst-case magnitudes
    codes = rng.integers(0, 4, (N, K), dtype=np.uint8)
    codes[0] = 3
    zp = rng.integers(0, 4, (K // g, N), dtype=np.uint8)
    zp[:, 0] = 0
    acc = oracle.c_gemm_acc(q, oracle.c_pack(codes), zp, g)
    np.testing.assert_array_equal(acc, oracle.np_gemm_acc_blas(q, codes, zp, g, np.float64))
    np.testing.assert_array_equal(acc, oracle.np_gemm_acc_blas(q, codes, zp, g, np.float32))
    assert acc[0, 0].max() == g * 127 * 3
    # torch CPU integer matmul, per group
    tq, tc = torch.from_numpy(q.astype(np.int32)), torch.from_numpy(codes.astype(np.int32))
    G = K // g
    raw = torch.einsum("mgk,ngk->mng", tq.reshape(M, G, g), tc.reshape(N, G, g)).numpy()
    rowsum = q.astype(np.int32).reshape(M, G, g).sum(axis=2)  # [M, G]
    folded = raw - zp.T.astype(np.int32)[None, :, :] * rowsum[:, None, :]
    np.testing.assert_array_equal(acc, folded)


# ------------------------------------------------------------------ epilogue
def test_epilogue_unit_scales_is_integer_sum(oracle):
    rng = np.random.default_rng(31)
    acc = rng.integers(-48768, 48769, (4, 6, 5)).astype(np.int32)
    ones = np.ones((5, 6), np.float16)
    s_a = np.array([1.0, 0.5, 2.0, 0.25], np.float32)
    bits, f32 = oracle.c_epilogue(acc, ones, s_a)
    np.testing.assert_array_equal(f32, acc.sum(axis=2).astype(np.float32) * s_a[:, None])
    np.testing.assert_array_equal(bits.view(np.float16), f32.astype(np.float16))


def test_epilogue_fma_chain_exact(oracle):
    """t_g = round32(acc_g * s_g + t_{g-1}) evaluated with exact rationals."""
    rng = np.random.default_rng(32)
    M, N, G = 2, 3, 6
    acc = rng.integers(-3000, 3000, (M, N, G)).astype(np.int32)
    scales = (rng.uniform(0.005, 0.02, (G, N))).astype(np.float16)
    s_a = rng.uniform(0.01, 0.05, M).astype(np.float32)
    _, f32 = oracle.c_epilogue(acc, scales, s_a)
    for m in range(M):
        for n in range(N):
            t = Fraction(0)
            for gi in range(G):
                exact = Fraction(int(acc[m, n, gi])) * Fraction(float(scales[gi, n])) + t
                as64 = float(exact)
                assert Fraction(as64) == exact  # representable in binary64: one rounding below
                t = Fraction(float(np.float32(as64)))
            want = np.float32(np.float32(float(t)) * s_a[m])
            assert f32[m, n] == want


def test_epilogue_close_to_float64(oracle):
    rng = np.random.default_rng(33)
    M, N, G = 8, 64, 32
    acc = rng.integers(-5000, 5000, (M, N, G)).astype(np.int32)
    scales = rng.uniform(0.001, 0.03, (G, N)).astype(np.float16)
    s_a = rng.uniform(0.01, 0.05, M).astype(np.float32)
    bits, f32 = oracle.c_epilogue(acc, scales, s_a)
    ref = oracle.np_epilogue_f64(acc, scales, s_a)
    scale_mag = np.abs(acc).astype(np.float64).sum(axis=2) * 0.03 * s_a[:, None]
    assert np.all(np.abs(f32 - ref) <= 2.0 ** -21 * scale_mag)
    bb, _ = oracle.c_epilogue(acc, scales, s_a, out_bf16=True)
    np.testing.assert_array_equal(bb, oracle.f32_to_bf16_bits(f32))


def test_fused_equals_two_step(oracle):
    rng = np.random.default_rng(34)
    M, N, K, g = 5, 33, 256, 64
    q = rng.integers(-127, 128, (M, K), dtype=np.int8)
    packed = rng.integers(0, 256, (N, K // 4), dtype=np.uint8)
    zp = rng.integers(0, 4, (K // g, N), dtype=np.uint8)
    scales = rng.uniform(0.001, 0.03, (K // g, N)).astype(np.float16)
    s_a = rng.uniform(0.01, 0.05, M).astype(np.float32)
    acc = oracle.c_gemm_acc(q, packed, zp, g)
    bits, _ = oracle.c_epilogue(acc, scales, s_a)
    fbits, fsum = oracle.c_gemm_fused(q, s_a, packed, scales, zp, g, want_acc_sum=True)
    np.testing.assert_array_equal(bits, fbits)
    np.testing.assert_array_equal(fsum, acc.sum(axis=2))
