"""The weight-only form (fp16 or bf16 activations times 2-bit weights on the fp16 resp. bf16 matrix cores).

Upstream's sketch is the notebook kernel ``w2matmul`` (slimkernels/triton/gemm_splitk.ipynb cell 1): 2-bit
fields widened to fp16 in front of an fp32-accumulating ``tl.dot``; it carries no scales and no zero-point and has
no test or stored output, so there is nothing of upstream's to compare numbers with.  The result is floating
point: the GPU path is held to the float64 restatement within max(1 ULP of the output type, rtol 1e-3,
2^-17 * sum of the terms' magnitudes) -- the last admits fp32 summation in the kernel's order and is far below
what one dropped or misplaced term would change (1 / K of that sum)."""
import ctypes

import numpy as np
import pytest
import torch

from slimkernels_amd import _lib, workloads
import parity_utils as pu

FAKE = 0x10000


def _weights(N, K, g, mode, seed):
    case = pu.small_case(1, N, K, g, mode, seed)
    packed, scales, zero = pu.quantized_weight(case)
    return case, packed, scales, zero


# ---------------------------------------------------------------- the oracle itself

def test_oracle_by_hand():
    from oracle import w2a8_oracle as o
    # one token row, two channels, K = 4, one group: codes - zp = [-2, -1, 0, 1] and [1, 1, -2, 0]
    x = np.array([[1.0, 2.0, -3.0, 0.5]], np.float16)
    codes = np.array([[0, 1, 2, 3], [3, 3, 0, 2]], np.uint8)
    scales = np.array([[0.5, 2.0]], np.float16)
    zp = np.array([[2, 2]], np.uint8)
    out, mag = o.w2a16_reference_forward(x, codes, scales, zp, 4)
    assert out.tolist() == [[0.5 * (-2 - 2 + 0 + 0.5), 2.0 * (1 + 2 + 6 + 0)]]
    assert mag.tolist() == [[0.5 * (2 + 2 + 0 + 0.5), 2.0 * (1 + 2 + 6 + 0)]]


@pytest.mark.parametrize("mode", ["sym", "asym"])
def test_oracle_against_a_library_matmul_and_plain_loops(mode):
    from oracle import w2a8_oracle as o
    case, packed, scales, zero = _weights(48, 256, 64, mode, seed=5)
    codes = o.np_unpack(packed)
    x = workloads.make_activation(pu.small_case(3, 48, 256, 64, mode, 5))
    out, _ = o.w2a16_reference_forward(x, codes, scales, zero, 64)
    # the dequantised weight times the activations through torch's matmul, in float64
    deq = (codes.astype(np.float64) - np.repeat(zero.T.astype(np.float64), 64, axis=1)) * \
        np.repeat(scales.T.astype(np.float64), 64, axis=1)
    want = torch.from_numpy(x.astype(np.float64)) @ torch.from_numpy(deq).T
    np.testing.assert_allclose(out, want.numpy(), rtol=1e-12, atol=1e-12)
    # a few elements by plain Python loops
    for m, n in ((0, 0), (2, 47), (1, 17)):
        acc = 0.0
        for k in range(256):
            acc += float(x[m, k]) * (int(codes[n, k]) - int(zero[k // 64, n])) * float(scales[k // 64, n])
        assert abs(acc - out[m, n]) <= 1e-9 * max(1.0, abs(acc))


# ---------------------------------------------------------------- host side of the entry point

def test_w2a16_validation():
    L = _lib.lib()
    g = L.slimk_w2a16_gemm
    # (x, ldx, x_dtype, w_r, s_r, zp_r, zp_const, M, N, K, group, out, ldo, out_dtype, ws, ws_bytes, split, stream)
    ok = [FAKE, 4096, 0, FAKE, FAKE, None, 2, 1, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 1, None]

    def call(**kw):
        names = ["x", "ldx", "xdt", "w", "s", "zp", "zpc", "M", "N", "K", "g", "out", "ldo", "odt", "ws", "wsb", "split", "st"]
        a = list(ok)
        for k, v in kw.items():
            a[names.index(k)] = v
        return g(*a)

    assert call(x=None) == 1
    assert call(M=0) == 2
    assert call(K=4096 + 64, ldx=4160, g=64) == 7 and b"multiple of 128" in L.slimk_w2a8_last_error()
    assert call(xdt=2) == 4 and call(odt=5) == 4                          # fp16 (0) and bf16 (1) activations only
    assert call(zpc=4) == 2
    assert call(ldx=4000) == 2 and call(ldo=100) == 2
    assert call(ldx=4100) == 3 and call(x=FAKE + 2) == 3
    assert call(g=100) == 2
    assert call(split=4) == 5 and b"workspace" in L.slimk_w2a8_last_error()
    assert call(split=4, ws=FAKE, wsb=1024) == 5
    assert call(split=65) == 2 and call(K=256, ldx=256, split=2) == 2     # more K-parts than there is K
    assert call(M=1 << 20, ldx=4096) == 7                                 # 32-bit offsets


def test_w2a16_split_and_workspace():
    L = _lib.lib()
    assert L.slimk_w2a16_gemm_auto_split_k(1, 28672, 8192, 128) >= 1
    for M, N, K, g in ((1, 4096, 4096, 128), (16, 28672, 8192, 128), (4, 256, 256, 64), (1, 14336, 4096, 256)):
        s = L.slimk_w2a16_gemm_auto_split_k(M, N, K, g)
        granules = K // max(g, 128)
        assert 1 <= s <= 64 and (s == 1 or s * 4 <= granules)
        assert L.slimk_w2a16_gemm_workspace_bytes(M, N, K, g, 0) == (0 if s == 1 else s * M * N * 4)
        assert L.slimk_w2a16_gemm_workspace_bytes(M, N, K, g, 3) == 3 * M * N * 4
    assert L.slimk_w2a16_gemm_auto_split_k(1, 4096, 4096 + 64, 64) == 0   # K not a multiple of 128


# ---------------------------------------------------------------- the GPU path against the oracle

def _check(got: torch.Tensor, want, mag, bf16, what):
    g = pu.bits_to_f32(pu.out_tensor_bits(got), bf16).astype(np.float64)
    assert np.isfinite(g).all(), f"{what}: non-finite output"
    tol = np.maximum(np.maximum(pu.ulp_of(want.astype(np.float32), bf16), 1e-3 * np.abs(want)), 2.0 ** -17 * mag)
    diff = np.abs(g - want)
    bad = diff > tol
    assert not bad.any(), (f"{what}: {int(bad.sum())} of {bad.size} outputs off; worst |diff|/tol = "
                           f"{float((diff / tol).max()):.3g} at {np.unravel_index(np.argmax(diff / tol), diff.shape)}")


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,g,mode,out,split", [
    (1, 256, 256, 128, "sym", "float16", 0),
    (1, 4096, 4096, 128, "sym", "float16", 0),
    (3, 200, 512, 64, "asym", "float16", 1),       # N not a multiple of 64, per-group zero-points, group 64
    (16, 1024, 2048, 128, "asym", "bfloat16", 0),
    (5, 320, 2048, 256, "sym", "float16", 2),      # group 256: a group spans two loop iterations
    (7, 192, 1792, 64, "sym", "bfloat16", 3),      # K-parts of unequal length
    (16, 128, 128, 64, "asym", "float16", 1),      # three of the four K-parts of a workgroup are empty
    (40, 448, 1024, 128, "ref", "float16", 0),     # several blocks of 16 token rows, uniform zero-point 1
    (2, 14336, 4096, 128, "sym", "float16", 0),
])
def test_w2a16_gemm_against_the_oracle(gpu_ops, oracle, M, N, K, g, mode, out, split):
    print(f"W2A16 M={M} N={N} K={K} g={g} {mode} {out} split={split}", flush=True)
    case = pu.small_case(M, N, K, g, mode, seed=M * 7 + N, out_dtype=out)
    packed, scales, zero = pu.quantized_weight(case)
    x = workloads.make_activation(case)
    want, mag = oracle.w2a16_reference_forward(x, oracle.np_unpack(packed), scales, zero, g)
    w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
    y = gpu_ops.w2a16_gemm(xd, w, pu.torch_dtype(case), split_k=split)
    assert y.shape == (M, N)
    _check(y, want, mag, out == "bfloat16", "W2A16")
    # a second call (the partial-sum buffer is reused) and a strided activation give the same bits
    wide = torch.zeros((M, K + 64), dtype=torch.float16, device="cuda")
    wide[:, :K] = xd
    y2 = gpu_ops.w2a16_gemm(wide[:, :K], w, pu.torch_dtype(case), split_k=split)
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,g,mode,out,split", [
    (1, 4096, 4096, 128, "sym", "bfloat16", 0),
    (3, 200, 512, 64, "asym", "bfloat16", 1),      # N not a multiple of 64, per-group zero-points, group 64
    (16, 1024, 2048, 128, "asym", "float16", 0),
    (5, 320, 2048, 256, "sym", "bfloat16", 2),     # group 256: a group spans two loop iterations
    (7, 192, 1792, 64, "ref", "bfloat16", 3),      # K-parts of unequal length, uniform zero-point 1
    (40, 448, 1024, 128, "sym", "bfloat16", 0),    # several blocks of 16 token rows
    (2, 14336, 4096, 128, "sym", "bfloat16", 0),
])
def test_w2a16_gemm_with_bf16_activations_against_the_oracle(gpu_ops, oracle, M, N, K, g, mode, out, split):
    """bf16 activations as they are (the bf16 matrix cores; the codes enter as 1 + code / 4 and the group's activation sum
    takes the offset and the zero-point off): the oracle's float64 result from the same bf16 values, to the tolerance
    of the fp16 form.  A row of large activations with a non-zero mean is the case that costs this form bits."""
    print(f"W2A16 bf16 activations M={M} N={N} K={K} g={g} {mode} {out} split={split}", flush=True)
    case = pu.small_case(M, N, K, g, mode, seed=M * 11 + N, out_dtype=out)
    packed, scales, zero = pu.quantized_weight(case)
    x = workloads.make_activation(case).astype(np.float32)
    x[0] = x[0] * 30.0 + 17.0                                             # large, far from zero mean
    w, _ = pu.device_inputs(gpu_ops, case, packed, scales, zero, workloads.make_activation(case))
    xd = torch.from_numpy(x).cuda().to(torch.bfloat16)
    x_bits = xd.view(torch.int16).cpu().numpy().view(np.uint16)
    want, mag = oracle.w2a16_reference_forward(x_bits, oracle.np_unpack(packed), scales, zero, g, x_bf16=True)
    y = gpu_ops.w2a16_gemm(xd, w, pu.torch_dtype(case), split_k=split)
    assert y.shape == (M, N)
    _check(y, want, mag, out == "bfloat16", "W2A16 bf16 activations")
    y2 = gpu_ops.w2a16_gemm(xd.clone(), w, pu.torch_dtype(case), split_k=split)
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))


@pytest.mark.gpu
def test_w2a16_linear_layer_keeps_bf16_activations(gpu_ops, oracle):
    case = pu.small_case(6, 256, 512, 128, "asym", seed=31, out_dtype="bfloat16")
    packed, scales, zero = pu.quantized_weight(case)
    w, _ = pu.device_inputs(gpu_ops, case, packed, scales, zero, workloads.make_activation(case))
    layer = gpu_ops.W2A16Linear(w, out_dtype=torch.bfloat16)
    x = torch.randn(2, 3, 512, device="cuda").to(torch.bfloat16)
    y = layer(x)
    x_bits = x.reshape(6, 512).view(torch.int16).cpu().numpy().view(np.uint16)
    want, mag = oracle.w2a16_reference_forward(x_bits, oracle.np_unpack(packed), scales, zero, 128, x_bf16=True)
    assert y.shape == (2, 3, 256) and y.dtype == torch.bfloat16
    _check(y.reshape(6, 256), want, mag, True, "W2A16Linear bf16")


def test_w2a16_grouped_validation():
    L = _lib.lib()
    P = _lib.Problem16
    def arr(*ps):
        a = (P * len(ps))(*ps)
        return ctypes.byref(a), len(ps)
    ok = dict(x=FAKE, w_r=FAKE, s_r=FAKE, zp_r=None, out=FAKE, ldx=4096, ldo=4096, M=1, N=4096, K=4096, zp_const=2)
    def prob(**kw):
        d = dict(ok); d.update(kw)
        return P(d["x"], d["w_r"], d["s_r"], d["zp_r"], d["out"], d["ldx"], d["ldo"], d["M"], d["N"], d["K"], d["zp_const"])
    g = L.slimk_w2a16_gemm_grouped
    a, n = arr(prob())
    assert g(None, 1, 128, 0, 0, None) == 1
    assert g(a, 0, 128, 0, 0, None) == 2 and g(a, 25, 128, 0, 0, None) == 2
    assert g(a, n, 128, 2, 0, None) == 4 and g(a, n, 128, 0, 3, None) == 4 and g(a, n, 100, 0, 0, None) == 2
    for bad, code in ((dict(x=None), 1), (dict(M=0), 2), (dict(K=4096 + 64, ldx=4160), 7), (dict(ldx=4000), 2), (dict(ldo=8), 2),
                      (dict(x=FAKE + 2), 3), (dict(ldx=4100), 3), (dict(zp_const=4), 2)):
        a, n = arr(prob(), prob(**bad))
        assert g(a, n, 64, 0, 0, None) == code, (bad, L.slimk_w2a8_last_error())
    a, n = arr(prob(), prob(zp_r=FAKE))
    assert g(a, n, 128, 1, 1, None) == 7 and b"mix" in L.slimk_w2a8_last_error()


@pytest.mark.gpu
@pytest.mark.parametrize("xdt,mode,out,g", [("float16", "sym", "float16", 128), ("bfloat16", "asym", "bfloat16", 64),
                                             ("bfloat16", "ref", "float16", 256), ("float16", "asym", "bfloat16", 128)])
def test_w2a16_grouped_launch_against_the_oracle(gpu_ops, oracle, xdt, mode, out, g):
    """Problems of different M, N (ragged) and K in one launch: every output against the oracle to the single launch's
    tolerance, a second launch bit-identical, and a launch of one problem."""
    shapes = [(1, 512, 1024), (3, 200, 512), (16, 1000, 2048), (17, 64, 256), (40, 320, 1536), (2, 4096, 4096)]
    dt = torch.bfloat16 if xdt == "bfloat16" else torch.float16
    odt = torch.bfloat16 if out == "bfloat16" else torch.float16
    probs, wants = [], []
    for i, (M, N, K) in enumerate(shapes):
        case = pu.small_case(M, N, K, g, mode, seed=500 + i, out_dtype=out)
        packed, scales, zero = pu.quantized_weight(case)
        w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, workloads.make_activation(case))
        xd = (xd.float() + (0.5 if i % 2 else 0.0)).to(dt)
        x_np = xd.view(torch.int16).cpu().numpy().view(np.uint16) if dt == torch.bfloat16 else xd.cpu().numpy()
        wants.append(oracle.w2a16_reference_forward(x_np, oracle.np_unpack(packed), scales, zero, g, x_bf16=dt == torch.bfloat16))
        probs.append((xd, w))
    outs = gpu_ops.w2a16_gemm_grouped(probs, odt)
    torch.cuda.synchronize()
    for i, (y, (want, mag)) in enumerate(zip(outs, wants)):
        assert y.shape == (shapes[i][0], shapes[i][1]) and y.dtype == odt
        _check(y, want, mag, out == "bfloat16", f"W2A16 grouped problem {i} {shapes[i]}")
    again = gpu_ops.w2a16_gemm_grouped(probs, odt)
    assert all(torch.equal(a.view(torch.int16), b.view(torch.int16)) for a, b in zip(outs, again))
    one = gpu_ops.w2a16_gemm_grouped(probs[2:3], odt)
    _check(one[0], wants[2][0], wants[2][1], out == "bfloat16", "W2A16 grouped launch of one problem")
    with pytest.raises(ValueError):
        gpu_ops.w2a16_gemm_grouped([probs[0], (probs[1][0].to(torch.float16 if dt == torch.bfloat16 else torch.bfloat16), probs[1][1])], odt)


@pytest.mark.gpu
def test_w2a16_agrees_with_the_int8_path_to_the_activation_quantisation(gpu_ops):
    """Same weights, same activations: the W2A8 result differs from the weight-only one only by the int8
    rounding of the activations (per-token scale absmax / 127: relative error of a sum of K terms ~ 1 %)."""
    case = pu.small_case(4, 512, 2048, 128, "sym", seed=3)
    packed, scales, zero = pu.quantized_weight(case)
    w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, workloads.make_activation(case))
    a16 = gpu_ops.w2a16_gemm(xd, w).float()
    a8 = gpu_ops.w2a8_gemm(gpu_ops.quantize_act_int8(xd, 128), w).float()
    err = (a16 - a8).norm() / a16.norm()
    print(f"relative L2 difference W2A16 vs W2A8: {err:.4f}", flush=True)
    assert 0 < err < 0.03


@pytest.mark.gpu
def test_w2a16_linear_layer(gpu_ops, oracle):
    """W2A16Linear against the float64 product with the dequantised weight, bias included, leading dimensions kept."""
    from slimkernels_amd.quantization import prepare_w2
    rng = np.random.default_rng(21)
    w = (rng.standard_normal((192, 512)) * 0.02).astype(np.float32)
    bias = torch.from_numpy(rng.standard_normal(192).astype(np.float16)).cuda()
    lin = gpu_ops.W2A16Linear.from_float(w, 128, "sym", bias=bias)
    packed, scales, zero = prepare_w2(w, 128, "sym")
    x = rng.standard_normal((2, 3, 512)).astype(np.float16)
    want, mag = oracle.w2a16_reference_forward(x.reshape(6, 512), oracle.np_unpack(packed), scales, zero, 128)
    y = lin(torch.from_numpy(x).cuda())
    assert y.shape == (2, 3, 192)
    got = y.reshape(6, 192).float().cpu().numpy().astype(np.float64)
    want = want + bias.float().cpu().numpy().astype(np.float64)[None, :]
    tol = np.maximum(2e-3 * np.abs(want), 2.0 ** -17 * mag) + 2.0 ** -10 * np.abs(bias.float().cpu().numpy())[None, :] + 1e-4
    assert (np.abs(got - want) <= tol).all(), float((np.abs(got - want) / tol).max())


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_w2a16_seeded_random_shapes(gpu_ops, oracle, seed):
    """Ten drawn shapes per seed: ragged N, 1..40 token rows, K any multiple of 128 the group divides, all three group
    sizes, every zero-point mode, both output types, forced and automatic K splits (a split the entry point refuses
    for the shape is checked to be refused, not run)."""
    rng = np.random.default_rng(1000 + seed)
    for i in range(10):
        g = int(rng.choice([64, 128, 256]))
        K = int(rng.integers(1, 17)) * 256 if g == 256 else int(rng.integers(1, 33)) * 128
        N = int(rng.integers(1, 700))
        M = int(rng.choice([1, 2, 3, 4, 7, 16, 17, 33, 40]))
        mode = str(rng.choice(["sym", "asym", "ref"]))
        out = str(rng.choice(["float16", "bfloat16"]))
        split = int(rng.choice([0, 0, 1, 2, 3, 5]))
        print(f"W2A16 random seed={seed} #{i}: M={M} N={N} K={K} g={g} {mode} {out} split={split}", flush=True)
        case = pu.small_case(M, N, K, g, mode, seed=seed * 100 + i, out_dtype=out)
        packed, scales, zero = pu.quantized_weight(case)
        x = workloads.make_activation(case)
        w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
        granules = K // max(g, 128)
        if split > 1 and split * 4 > granules:
            with pytest.raises(_lib.SlimkError):
                gpu_ops.w2a16_gemm(xd, w, pu.torch_dtype(case), split_k=split)
            continue
        want, mag = oracle.w2a16_reference_forward(x, oracle.np_unpack(packed), scales, zero, g)
        y = gpu_ops.w2a16_gemm(xd, w, pu.torch_dtype(case), split_k=split)
        _check(y, want, mag, out == "bfloat16", f"W2A16 seed {seed} case {i}")
        # the same draw as bf16 activations (rounded from the fp16 values, shifted off zero mean in every other case)
        xb = (xd.float() + (0.75 if i % 2 else 0.0)).to(torch.bfloat16)
        x_bits = xb.view(torch.int16).cpu().numpy().view(np.uint16)
        want, mag = oracle.w2a16_reference_forward(x_bits, oracle.np_unpack(packed), scales, zero, g, x_bf16=True)
        y = gpu_ops.w2a16_gemm(xb, w, pu.torch_dtype(case), split_k=split)
        _check(y, want, mag, out == "bfloat16", f"W2A16 bf16 activations seed {seed} case {i}")


@pytest.mark.gpu
def test_wrappers_take_awkward_activation_views(gpu_ops):
    """Activations that the C entry points would refuse (row pitch not a multiple of 8, rows broadcast with pitch 0,
    a start that is not 16-byte aligned) are copied by the wrappers: same bits as from a plain tensor."""
    case = pu.small_case(3, 256, 512, 128, "sym", seed=9)
    packed, scales, zero = pu.quantized_weight(case)
    w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, workloads.make_activation(case))
    pitch = torch.zeros((3, 516), dtype=torch.float16, device="cuda")
    pitch[:, :512] = xd
    shifted = torch.zeros((3 * 512 + 1,), dtype=torch.float16, device="cuda")
    shifted[1:] = xd.reshape(-1)
    views = {"pitch 516": pitch[:, :512], "offset 2 bytes": shifted[1:].reshape(3, 512)}
    for what, v in views.items():
        assert torch.equal(gpu_ops.w2a16_gemm(v, w), gpu_ops.w2a16_gemm(xd, w)), what
        a, b = gpu_ops.quantize_act_int8(v, 128), gpu_ops.quantize_act_int8(xd, 128)
        assert torch.equal(a.q, b.q) and torch.equal(a.s_a, b.s_a), what
    row = xd[:1].expand(3, 512)                                   # pitch 0
    y = gpu_ops.w2a16_gemm(row, w)
    assert torch.equal(y[0], y[1]) and torch.equal(y[0], gpu_ops.w2a16_gemm(xd[:1], w)[0])
    one = gpu_ops.w2a8_linear_fused(shifted[1:513].reshape(1, 512), w)
    assert torch.equal(one, gpu_ops.w2a8_linear_fused(xd[:1].contiguous(), w))
