"""W4A8: 4-bit weights run as two 2-bit planes through the W2A8 kernels.

Upstream's W4 code is one notebook kernel on random packed integers (slimkernels/triton/gemm_splitk.ipynb
cell 0) with no quantiser and no tests, so there are no upstream vectors to carry over: the host functions
are pinned by hand-computed cases, closed forms, brute force and the notebook's unpack expression, and the GPU
path by the oracle's exact integer sums and its epilogue (the tolerance of the W2 path, written in
parity_utils.assert_out_close: 1 ULP of the output type or rtol 1e-3, plus the fp32 re-association bound)."""
import numpy as np
import pytest
import torch

from slimkernels_amd import w4
import parity_utils as pu


# ---------------------------------------------------------------- host format and quantiser (CPU)

def test_pack_w4_known_answer_and_round_trip():
    codes = np.array([[1, 2, 15, 0], [8, 8, 3, 12]], dtype=np.uint8)
    packed = w4.pack_w4(codes)
    np.testing.assert_array_equal(packed, np.array([[0x12, 0xF0], [0x88, 0x3C]], dtype=np.uint8))
    np.testing.assert_array_equal(w4.unpack_w4(packed), codes)
    every = np.arange(256, dtype=np.uint8).reshape(1, 256)
    np.testing.assert_array_equal(w4.pack_w4(w4.unpack_w4(every)), every)


def test_pack_w4_rejects_bad_input():
    with pytest.raises(ValueError):
        w4.pack_w4(np.zeros((2, 4), dtype=np.int32))
    with pytest.raises(ValueError):
        w4.pack_w4(np.zeros((2, 3), dtype=np.uint8))
    with pytest.raises(ValueError):
        w4.pack_w4(np.full((2, 4), 16, dtype=np.uint8))


def test_uint32_operand_of_the_notebook(oracle):
    rng = np.random.default_rng(0)
    b = rng.integers(0, 2**32, size=(4, 5), dtype=np.uint64).astype(np.uint32)   # K = 32, N = 5
    codes = w4.codes_from_uint32_kn(b)
    assert codes.shape == (5, 32) and codes.dtype == np.uint8
    for n in range(5):           # the notebook's expression, element by element
        for k in range(32):
            assert codes[n, k] == (int(b[k // 8, n]) >> ((k % 8) * 4)) & 0xF
    np.testing.assert_array_equal(codes, oracle.np_unpack_uint32_kn(b))
    np.testing.assert_array_equal(w4.codes_from_uint32_kn(b.view(np.int32)), codes)   # signed storage, same bits


def test_quantize_w4_sym_closed_form():
    # one group of 8 rows, two columns; absmax 4 -> s = 0.5, codes = rne(w / 0.5) + 8 clipped to 0..15
    col0 = np.array([-4.0, -3.75, -0.25, 0.0, 0.25, 0.75, 3.4, 4.0], dtype=np.float32)
    col1 = col0[::-1] * 2
    codes, scales, zp = w4.quantize_w4(np.stack([col0, col1], axis=1), group_size=8, mode="sym")
    np.testing.assert_array_equal(scales, np.array([[0.5, 1.0]], dtype=np.float32))
    np.testing.assert_array_equal(zp, np.array([[8, 8]], dtype=np.uint8))
    # -4 -> 0; -3.75/0.5 = -7.5 -> -8 (ties to even) -> 0; -0.25/0.5 = -0.5 -> -0 -> 8; 0.25/0.5 = 0.5 -> 0 -> 8;
    # 0.75/0.5 = 1.5 -> 2 -> 10; 3.4/0.5 = 6.8 -> 7 -> 15; 4/0.5 = 8 -> 16 clipped to 15
    np.testing.assert_array_equal(codes[:, 0], np.array([0, 0, 8, 8, 8, 10, 15, 15], dtype=np.uint8))
    np.testing.assert_array_equal(codes[:, 1], codes[::-1, 0])


@pytest.mark.parametrize("mode", ["sym", "asym"])
def test_quantize_w4_against_brute_force_and_the_oracle(oracle, mode):
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((64, 6)) * 0.05).astype(np.float32)
    w[5, 2] = 0.0
    codes, scales, zp = w4.quantize_w4(w, group_size=16, mode=mode)
    oc, os_, oz = oracle.np_quantize_w4(w, 16, mode)
    np.testing.assert_array_equal(codes, oc)
    np.testing.assert_array_equal(scales, os_)
    np.testing.assert_array_equal(zp, oz)
    for g in range(4):           # scalar restatement, element by element
        for n in range(6):
            col = w[16 * g:16 * g + 16, n]
            if mode == "sym":
                s = np.float32(max(np.abs(col).max(), np.float32(1e-9))) / np.float32(8.0)
                z = 8
            else:
                s = np.float32(max(col.max() - col.min(), np.float32(1e-9))) / np.float32(15.0)
                z = int(np.clip(np.round(np.float32(-col.min()) / s), 0, 15))
            assert scales[g, n] == s and zp[g, n] == z
            for i, v in enumerate(col):
                assert codes[16 * g + i, n] == int(np.clip(np.round(np.float32(v) / s) + z, 0, 15))
    # every level is within half a step of the value it stands for, inside the clip range
    deq = (codes.astype(np.float32).reshape(4, 16, 6) - zp[:, None, :]) * scales[:, None, :]
    inside = (codes > 0) & (codes < 15)
    assert np.all(np.abs(deq.reshape(64, 6) - w)[inside] <= np.repeat(scales, 16, axis=0)[inside] * 0.5 + 1e-9)


def test_split_planes_identity():
    rng = np.random.default_rng(5)
    N, K, g = 7, 256, 64
    codes = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    scales = (rng.random((K // g, N)) * 0.01 + 0.001).astype(np.float16)
    zp = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    packed2, scales2, zp2 = w4.split_planes(codes, scales, zp)
    from slimkernels_amd import unpack_matrix
    planes = unpack_matrix(packed2)
    assert planes.shape == (N, 2 * K) and scales2.shape == (2 * K // g, N) and zp2.max() <= 3
    np.testing.assert_array_equal(planes[:, :K].astype(np.int32) * 4 + planes[:, K:], codes)
    np.testing.assert_array_equal(zp2[:K // g].astype(np.int32) * 4 + zp2[K // g:], zp)
    np.testing.assert_array_equal(scales2[K // g:], scales)
    np.testing.assert_array_equal(scales2[:K // g].astype(np.float32), scales.astype(np.float32) * 4)
    # the identity the GPU path rests on, on integers: sum q (c - zp) = 4 sum q (hi - zh) + sum q (lo - zl)
    q = rng.integers(-127, 128, size=(3, K)).astype(np.int64)
    for gi in range(K // g):
        ks = slice(gi * g, (gi + 1) * g)
        want = q[:, ks] @ (codes[:, ks].astype(np.int64) - zp[gi][:, None]).T
        hi = q[:, ks] @ (planes[:, :K][:, ks].astype(np.int64) - zp2[gi][:, None]).T
        lo = q[:, ks] @ (planes[:, K:][:, ks].astype(np.int64) - zp2[K // g + gi][:, None]).T
        np.testing.assert_array_equal(4 * hi + lo, want)
    with pytest.raises(ValueError, match="overflows"):
        w4.split_planes(codes, np.full_like(scales, 30000.0), zp)


# ---------------------------------------------------------------- the GPU path

def _plane_bound(oracle, ref, codes, scales, zp, g):
    """The fp32 re-association bound of the sum as the GPU forms it: 2G terms per output, the hi-plane sums
    times 4 * scale and the lo-plane sums times scale (a plane's term can be larger than their sum)."""
    hi = oracle.np_gemm_acc_blas(ref["q"], codes >> 2, zp >> 2, g)
    lo = oracle.np_gemm_acc_blas(ref["q"], codes & 3, zp & 3, g)
    np.testing.assert_array_equal(4 * hi + lo, ref["acc"])
    return pu.reorder_bound(np.concatenate([4 * hi, lo], axis=2), np.concatenate([scales, scales], axis=0), ref["s_a"])


def _w4_case(M, N, K, g, mode, seed, outliers=False):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32) if mode == "sym" else \
        rng.uniform(-0.05, 0.05, size=(N, K)).astype(np.float32)
    x = rng.standard_normal((M, K)).astype(np.float32)
    if outliers:
        x[:, rng.choice(K, max(1, K // 1000), replace=False)] *= 20
    return w, x.astype(np.float16)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,g,mode,out,kernel", [
    (1, 256, 512, 128, "sym", "float16", "auto"),
    (5, 192, 256, 64, "asym", "float16", "skinny"),
    (16, 4096, 4096, 128, "sym", "float16", "auto"),
    (32, 1024, 2048, 128, "asym", "bfloat16", "auto"),
    (77, 320, 1024, 128, "asym", "float16", "tiled"),
    (256, 512, 1024, 128, "sym", "bfloat16", "auto"),
])
def test_w4a8_gemm_against_the_oracle(gpu_ops, oracle, M, N, K, g, mode, out, kernel):
    from slimkernels_amd.torch import w4 as tw4
    print(f"W4A8 M={M} N={N} K={K} g={g} {mode} {out} {kernel}", flush=True)
    w, x = _w4_case(M, N, K, g, mode, seed=M + N)
    packed4, scales, zp = w4.prepare_w4(w, g, mode)
    codes = w4.unpack_w4(packed4)
    bf16 = out == "bfloat16"
    ref = oracle.w4_reference_forward(x, codes, scales, zp, g, bf16)
    wd = tw4.repack_w4(packed4, scales, zp, g)
    qa = gpu_ops.quantize_act_int8(torch.from_numpy(x).cuda(), g)
    np.testing.assert_array_equal(qa.q.cpu().numpy(), ref["q"])
    odt = torch.bfloat16 if bf16 else torch.float16
    y, acc = tw4.w4a8_gemm(qa, wd, odt, kernel=kernel, dump="groups")
    np.testing.assert_array_equal(acc.cpu().numpy(), ref["acc"])          # int32 sums: exact
    y2 = tw4.w4a8_gemm(qa, wd, odt, kernel=kernel)
    bound = _plane_bound(oracle, ref, codes, scales, zp, g)
    for t, what in ((y, "with dump"), (y2, "production kernels")):
        pu.assert_out_close(pu.out_tensor_bits(t), ref["out_bits"], bf16, bound, f"W4A8 {what}")


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,g,bf16,copies", [(1, 1024, 128, False, 2), (5, 4096, 128, True, 2), (33, 8192, 64, False, 2),
                                                (7, 14336, 128, False, 2), (3, 20480, 128, True, 2), (2, 512, 64, False, 3)])
def test_act_quant_laid_down_several_times(gpu_ops, M, K, g, bf16, copies):
    """One launch that writes the quantised row and its group sums ``copies`` times gives exactly what the
    plain launch gives, repeated (all three kernels of the launcher: K <= 4096, <= 16384, beyond)."""
    print(f"act_quant copies: M={M} K={K} g={g} bf16={bf16} copies={copies}", flush=True)
    gen = torch.Generator().manual_seed(M * 131 + K)
    x = (torch.randn((M, K), generator=gen) * 3).to(torch.bfloat16 if bf16 else torch.float16).cuda()
    one = gpu_ops.quantize_act_int8(x, g)
    rep = gpu_ops.quantize_act_int8(x, g, copies=copies)
    assert rep.q.shape == (M, copies * K) and rep.rowsum.shape[0] == copies * (K // g)
    assert torch.equal(rep.q, torch.cat([one.q] * copies, dim=1))
    assert torch.equal(rep.rowsum[:, :M], torch.cat([one.rowsum[:, :M]] * copies, dim=0))
    assert torch.equal(rep.s_a, one.s_a)


@pytest.mark.gpu
def test_w4a8_linear_and_decode_row(gpu_ops, oracle):
    from slimkernels_amd.torch import w4 as tw4
    w, x = _w4_case(3, 384, 1024, 128, "sym", seed=11)
    lin = tw4.W4A8Linear.from_float(w, 128, "sym")
    packed4, scales, zp = w4.prepare_w4(w, 128, "sym")
    xd = torch.from_numpy(x).cuda()
    codes = w4.unpack_w4(packed4)
    ref = oracle.w4_reference_forward(x, codes, scales, zp, 128)
    bound = _plane_bound(oracle, ref, codes, scales, zp, 128)
    y = lin(xd.reshape(1, 3, 1024))
    assert y.shape == (1, 3, 384)
    pu.assert_out_close(pu.out_tensor_bits(y.reshape(3, 384)), ref["out_bits"], False, bound, "W4A8Linear")
    # one row: the single-launch kernel that quantises the row itself
    ref1 = oracle.w4_reference_forward(x[:1], codes, scales, zp, 128)
    y1 = lin(xd[:1])
    pu.assert_out_close(pu.out_tensor_bits(y1), ref1["out_bits"], False,
                        _plane_bound(oracle, ref1, codes, scales, zp, 128), "W4A8Linear one row")


@pytest.mark.gpu
def test_w4matmul_splitk_call_form(gpu_ops):
    """c += a @ codes with the notebook's operand layout; against the fp32 product of the same operands the
    only difference is the int8 quantisation of a (|error| <= s_a / 2 per element of a)."""
    from slimkernels_amd.torch import w4 as tw4
    rng = np.random.default_rng(2)
    M, N, K = 4, 64, 256
    a = rng.standard_normal((M, K)).astype(np.float16)
    b = rng.integers(0, 2**32, size=(K // 8, N), dtype=np.uint64).astype(np.uint32)
    codes = w4.codes_from_uint32_kn(b).astype(np.float32)                 # [N, K]
    c0 = rng.standard_normal((M, N)).astype(np.float16)
    c = torch.from_numpy(c0.copy()).cuda()
    out = tw4.w4matmul_splitk(torch.from_numpy(a).cuda(), torch.from_numpy(b.view(np.int32)), c)
    assert out is c
    want = c0.astype(np.float32) + a.astype(np.float32) @ codes.T
    s_a = np.abs(a.astype(np.float32)).max(axis=1) / 127
    tol = (s_a / 2)[:, None] * codes.sum(axis=1)[None, :] + 1e-3 * np.abs(want) + 0.26   # + fp16 rounding of c (|c| < 512)
    assert np.all(np.abs(c.float().cpu().numpy() - want) <= tol)


@pytest.mark.gpu
def test_w4_weight_through_the_file_container(gpu_ops, tmp_path):
    from slimkernels_amd.torch import w4 as tw4
    w, x = _w4_case(4, 192, 512, 128, "asym", seed=21)
    packed4, scales, zp = w4.prepare_w4(w, 128, "asym")
    path = str(tmp_path / "layer.w4")
    tw4.save_w4(path, packed4, scales, zp, 128)
    from_file = tw4.load_w4_weight(path)
    direct = tw4.repack_w4(packed4, scales, zp, 128)
    assert (from_file.N, from_file.K, from_file.group_size) == (192, 512, 128)
    assert torch.equal(from_file.planes.w_r, direct.planes.w_r) and torch.equal(from_file.planes.s_r, direct.planes.s_r)
    assert torch.equal(from_file.planes.zp_r, direct.planes.zp_r)
    xd = torch.from_numpy(x).cuda()
    assert torch.equal(tw4.w4a8_linear(xd, from_file), tw4.w4a8_linear(xd, direct))
    # a W2 file is not taken for a W4 one
    from slimkernels_amd import prepare_w2, save_w2
    p2, s2, _ = prepare_w2(w, 128, "sym")
    save_w2(str(tmp_path / "layer.w2"), p2, s2, None, 128, "sym")
    with pytest.raises(ValueError, match="not a two-plane W4 file"):
        tw4.load_w4_weight(str(tmp_path / "layer.w2"))


@pytest.mark.gpu
def test_w4a8_grouped_launch(gpu_ops, oracle):
    from slimkernels_amd.torch import w4 as tw4
    probs, refs = [], []
    for i, (M, N, K) in enumerate(((1, 512, 1024), (16, 320, 2048), (32, 256, 512), (5, 1000, 1024))):
        w, x = _w4_case(M, N, K, 128, "asym", seed=40 + i)
        packed4, scales, zp = w4.prepare_w4(w, 128, "asym")
        codes = w4.unpack_w4(packed4)
        ref = oracle.w4_reference_forward(x, codes, scales, zp, 128)
        qa = gpu_ops.quantize_act_int8(torch.from_numpy(x).cuda(), 128)
        out = torch.empty((M, N), dtype=torch.float16, device="cuda")
        probs.append((qa, tw4.repack_w4(packed4, scales, zp, 128), out))
        refs.append((ref, _plane_bound(oracle, ref, codes, scales, zp, 128)))
    tw4.w4a8_gemm_grouped(probs, torch.float16)
    torch.cuda.synchronize()
    for (_, _, out), (ref, bound) in zip(probs, refs):
        pu.assert_out_close(pu.out_tensor_bits(out), ref["out_bits"], False, bound, "W4A8 grouped")


@pytest.mark.gpu
@pytest.mark.parametrize("N,K,g,mode,bf16", [(64, 256, 64, "sym", False), (200, 1024, 128, "asym", False),
                                             (96, 2048, 256, "sym", True), (33, 4096, 128, "asym", True)])
def test_w4_quantisation_on_gpu_bit_exact(gpu_ops, N, K, g, mode, bf16):
    """The GPU 4-bit quantiser writes the two planes, their scales and zero-points exactly as the host functions
    do (prepare_w4 + split_planes); a group of equal values and an all-zero group are in the draw."""
    print(f"W4 quantise on GPU: N={N} K={K} g={g} {mode} bf16={bf16}", flush=True)
    rng = np.random.default_rng(N + K)
    wt = torch.from_numpy((rng.standard_normal((N, K)) * 0.05).astype(np.float32))
    wt[1, :g] = 0.0
    wt[2, g:2 * g] = 0.03125
    wt = wt.to(torch.bfloat16 if bf16 else torch.float16)
    planes, scales2, zp2 = gpu_ops.quantize_weight4_gpu(wt.cuda(), g, mode)
    packed4, scales, zero = w4.prepare_w4(wt.float().numpy(), g, mode)
    want_planes, want_scales, want_zp = w4.split_planes(w4.unpack_w4(packed4), scales, zero)
    assert np.array_equal(planes.cpu().numpy(), want_planes)
    assert np.array_equal(scales2.cpu().numpy().view(np.uint16), want_scales.view(np.uint16))
    assert np.array_equal(zp2.cpu().numpy(), want_zp)


@pytest.mark.gpu
def test_w4a8_linear_from_a_gpu_weight(gpu_ops):
    """from_float on a CUDA fp16 weight quantises on the GPU: same layer as from the host path, bit for bit."""
    from slimkernels_amd.torch import w4 as tw4
    w, x = _w4_case(5, 192, 512, 128, "asym", seed=4)
    w16 = torch.from_numpy(w).half()
    a = tw4.W4A8Linear.from_float(w16.cuda(), 128, "asym")
    b = tw4.W4A8Linear.from_float(w16.float().numpy(), 128, "asym")
    assert torch.equal(a.weight.planes.w_r, b.weight.planes.w_r) and torch.equal(a.weight.planes.s_r, b.weight.planes.s_r)
    assert torch.equal(a.weight.planes.zp_r, b.weight.planes.zp_r)
    xd = torch.from_numpy(x).cuda()
    assert torch.equal(a(xd), b(xd))


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,g,out,mode", [(64, 256, 512, 128, "float16", "sym"), (200, 320, 1024, 64, "float16", "sym"),
                                              (5, 100, 256, 128, "bfloat16", "sym"), (300, 1100, 2048, 128, "bfloat16", "sym"),
                                              (129, 64, 128, 64, "float16", "sym"), (200, 320, 1024, 64, "float16", "asym"),
                                              (77, 1100, 2048, 128, "bfloat16", "asym"), (40, 130, 4096, 128, "float16", "asym")])
def test_w4a8_one_pass_kernel(gpu_ops, oracle, M, N, K, g, out, mode):
    """Symmetric 4-bit weights through the kernel that joins the two digits in front of the matrix core: against the
    oracle (exact int32 sums, fp32 epilogue over G groups) to the output criterion of the path, ragged M and N."""
    from slimkernels_amd.torch import w4 as tw4
    print(f"W4A8 one pass M={M} N={N} K={K} g={g} {out} {mode}", flush=True)
    w, x = _w4_case(M, N, K, g, mode, seed=M + K)
    packed4, scales, zp = w4.prepare_w4(w, g, mode)
    codes = w4.unpack_w4(packed4)
    bf16 = out == "bfloat16"
    ref = oracle.w4_reference_forward(x, codes, scales, zp, g, out_bf16=bf16)
    w4d = tw4.repack_w4(packed4, scales, zp, g)
    assert w4d.uniform_zp8 == (mode == "sym")
    qa = gpu_ops.quantize_act_int8(torch.from_numpy(x).cuda(), g)
    dt = torch.bfloat16 if bf16 else torch.float16
    y = tw4.w4a8_gemm_one_pass(qa, w4d, dt)
    # per-group zero-points: a group's sum reaches the GPU's fp32 chain as two terms, sum q (code - 8) and
    # (8 - zp) * rowsum, each of which can be larger than their sum
    acc8 = oracle.np_gemm_acc_blas(ref["q"], codes, np.full_like(zp, 8), g)
    one_pass_bound = pu.reorder_bound(np.concatenate([acc8, ref["acc"] - acc8], axis=2), np.concatenate([scales, scales], axis=0),
                                      ref["s_a"])
    same = pu.assert_out_close(pu.out_tensor_bits(y), ref["out_bits"], bf16, one_pass_bound, "W4A8 one pass")
    print(f"  bit-identical with the oracle on {100 * same:.1f} % of the outputs", flush=True)
    # K split over several workgroups per tile: partial sums meet in the workspace in split order, so the result
    # is the same on every call and within the re-association bound of the oracle's
    for split in (2, 3):
        if split <= K // 128:
            ys = tw4.w4a8_gemm_one_pass(qa, w4d, dt, split_k=split)
            pu.assert_out_close(pu.out_tensor_bits(ys), ref["out_bits"], bf16, one_pass_bound, f"W4A8 one pass, split {split}")
            again = tw4.w4a8_gemm_one_pass(qa, w4d, dt, split_k=split)
            assert torch.equal(ys.view(torch.int16), again.view(torch.int16))
    y_after = tw4.w4a8_gemm_one_pass(qa, w4d, dt)          # the counters were left at zero
    assert torch.equal(y_after.view(torch.int16), y.view(torch.int16))
    bound = _plane_bound(oracle, ref, codes, scales, zp, g)
    # the layer takes this road from 33 token rows on and the two-plane road below
    lin = tw4.W4A8Linear(w4d, None, dt)
    y2 = lin(torch.from_numpy(x).cuda())
    pu.assert_out_close(pu.out_tensor_bits(y2), ref["out_bits"], bf16, bound, "W4A8Linear")
    assert tw4.one_pass_applies(M, w4d) == (M >= 33)
    if M >= 33:
        assert torch.equal(y2.view(torch.int16), y.view(torch.int16))


@pytest.mark.gpu
def test_w4_routes_share_one_workspace(gpu_ops, oracle):
    """The two-plane road (few rows: split-K skinny kernel over 2K) and the one-pass road (tiled kernel, K split over
    workgroups) of one weight object use the same workspace, in turn and with changing token counts: every result is
    the one a fresh weight object gives."""
    from slimkernels_amd.torch import w4 as tw4
    N, K, g = 256, 7168, 128
    w, _ = _w4_case(8, N, K, g, "sym", seed=77)
    packed4, scales, zp = w4.prepare_w4(w, g, "sym")
    shared = tw4.repack_w4(packed4, scales, zp, g)
    rng = np.random.default_rng(5)
    for M in (20, 64, 8, 200, 20, 40, 64):
        print("W4 workspace reuse M", M, flush=True)
        x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float16)).cuda()
        qa = gpu_ops.quantize_act_int8(x, g)
        fresh = tw4.repack_w4(packed4, scales, zp, g)
        if tw4.one_pass_applies(M, shared):
            got, want = tw4.w4a8_gemm_one_pass(qa, shared), tw4.w4a8_gemm_one_pass(qa, fresh)
        else:
            got, want = tw4.w4a8_gemm(qa, shared), tw4.w4a8_gemm(qa, fresh)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"M={M}"
    ws = shared.planes.workspace
    assert ws is not None and int(ws[:65536].view(torch.int32).abs().max()) == 0   # the counter block is back at zero


def test_one_pass_is_for_more_than_32_rows():
    from slimkernels_amd.torch import w4 as tw4
    big = dict(N=14336, K=4096, group_size=128)
    assert tw4.one_pass_applies(512, tw4.W4A8Weight(None, uniform_zp8=True, **big))
    assert tw4.one_pass_applies(33, tw4.W4A8Weight(None, uniform_zp8=False, **big))
    assert not tw4.one_pass_applies(32, tw4.W4A8Weight(None, uniform_zp8=True, **big))
    assert not tw4.one_pass_applies(4096, tw4.W4A8Weight(None, 14336, 4096, 256, uniform_zp8=True))
    assert not tw4.one_pass_applies(512, tw4.W4A8Weight(None, 4096, 4160, 64, uniform_zp8=True))      # K % 128
