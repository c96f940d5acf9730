"""CPU checks of the gfx950 streaming layout and of the kernels' index arithmetic."""
import numpy as np
import pytest

from slimkernels_amd import layout
from kernel_model import wave_strip_groups


@pytest.mark.parametrize("N,K", [(64, 64), (100, 128), (16, 256), (130, 192), (1, 64), (70, 576), (200, 1024)])
def test_repack_roundtrip(N, K):
    rng = np.random.default_rng(N * 1000 + K)
    packed = rng.integers(0, 256, (N, K // 4), dtype=np.uint8)
    w_r = layout.repack_codes(packed)
    assert w_r.shape == (-(-(K // 64) // 4), -(-N // 64), 4, 64, 4)
    assert not w_r.reshape(w_r.shape[0], w_r.shape[1], 4, 256)[-1, :, (K // 64 - 1) % 4 + 1:].any()   # padding units are zero
    np.testing.assert_array_equal(layout.unrepack_codes(w_r, N, K), packed)


def test_repack_field_definition():
    """Field p of byte b of dword i of lane (quad, col) is the code of (strip*64+p*16+col, step*64+quad*16+4i+b)."""
    rng = np.random.default_rng(1)
    N, K = 128, 128
    codes = rng.integers(0, 4, (N, K), dtype=np.uint8)
    q4 = codes.reshape(N, K // 4, 4)
    packed = ((q4[..., 0] << 6) | (q4[..., 1] << 4) | (q4[..., 2] << 2) | q4[..., 3]).astype(np.uint8)
    w_r = layout.repack_codes(packed)
    for _ in range(500):
        n, k = int(rng.integers(N)), int(rng.integers(K))
        strip, p, col = n // 64, (n % 64) // 16, n % 16
        step, quad, i, b = k // 64, (k % 64) // 16, (k % 16) // 4, k % 4
        f = (int(layout.unit(w_r, step, strip)[quad * 16 + col, i]) >> (8 * b + 2 * p)) & 3
        assert (f ^ 2 if p == 3 else f) == codes[n, k]


def test_group_value_layout():
    v = np.arange(3 * 70, dtype=np.float16).reshape(3, 70)
    r = layout.repack_group_values(v)
    assert r.shape == (3, 2, 16, 4)
    for n in (0, 15, 16, 63, 64, 69):
        for g in range(3):
            assert r[g, n // 64, n % 16, (n % 64) // 16] == v[g, n]
    assert r[0, 1, 6, 0] == 0  # n = 70 is padding


@pytest.mark.parametrize("mode,gs", [("sym", 2), ("asym", 1), ("asym", 2)])
def test_wave_model_matches_oracle(oracle, mode, gs):
    """Shift-free unpack + scaled zero-point folding + per-group drain == oracle accumulators."""
    rng = np.random.default_rng(40 + gs)
    M, N, g = 7, 64, 64 * gs
    K = g * 2
    x = rng.standard_normal((M, K)).astype(np.float16)
    q, s_a, rs = oracle.c_act_quant(x, g)
    packed = rng.integers(0, 256, (N, K // 4), dtype=np.uint8)
    scales = rng.uniform(0.005, 0.02, (K // g, N)).astype(np.float16)
    zp = rng.integers(0, 4, (K // g, N), dtype=np.uint8) if mode == "asym" else np.full((K // g, N), 2, np.uint8)
    acc = oracle.c_gemm_acc(q, packed, zp, g)
    _, out_f32 = oracle.c_epilogue(acc, scales, s_a)
    w_r = layout.repack_codes(packed)
    s_r = layout.repack_group_values(scales)
    zp_r = layout.repack_group_values(zp) if mode == "asym" else None
    rs_pad = np.zeros((K // g, 8), np.int32)
    rs_pad[:, :M] = rs
    t, acc_model = wave_strip_groups(q, rs_pad, w_r, s_r, zp_r, 2, 0, [0, 1], gs, M)
    np.testing.assert_array_equal(acc_model[:M], acc)
    np.testing.assert_allclose(t[:M] * s_a[:, None], out_f32, rtol=1e-6, atol=0)
