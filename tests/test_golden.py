"""Committed golden vectors (tests/golden/w2a8_small.npz): the oracle must still reproduce them
bit for bit (CPU), and so must the HIP kernels (GPU)."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "w2a8_small.npz")
MODES = {0: "ref", 1: "sym", 2: "asym"}


def _cases():
    z = np.load(GOLDEN)
    names = sorted({k.split("/")[0] for k in z.files})
    return z, names


def _get(z, name):
    d = {k.split("/")[1]: z[k] for k in z.files if k.startswith(name + "/")}
    M, N, K, g, mode, bf16 = (int(v) for v in d["meta"])
    return d, M, N, K, g, MODES[mode], bool(bf16)


def test_oracle_reproduces_golden(oracle):
    z, names = _cases()
    assert len(names) == 4
    for name in names:
        d, M, N, K, g, mode, bf16 = _get(z, name)
        x = d["x"].view(np.float16)
        q, s_a, rs = oracle.c_act_quant(x, g)
        np.testing.assert_array_equal(q, d["q"])
        np.testing.assert_array_equal(s_a, d["s_a"])
        np.testing.assert_array_equal(rs, d["rowsum"])
        acc = oracle.c_gemm_acc(q, d["packed"], d["zp"], g)
        np.testing.assert_array_equal(acc, d["acc"])
        np.testing.assert_array_equal(acc, oracle.np_gemm_acc_blas(q, oracle.np_unpack(d["packed"]), d["zp"], g))
        bits, _ = oracle.c_epilogue(acc, d["scales"].view(np.float16), s_a, bf16)
        np.testing.assert_array_equal(bits, d["out_bits"])
        fused, _ = oracle.c_gemm_fused(q, s_a, d["packed"], d["scales"].view(np.float16), d["zp"], g, bf16)
        np.testing.assert_array_equal(fused, d["out_bits"])


def test_host_quantizer_reproduces_golden_weights():
    """The packed codes / scales / zero-points in the fixture come from the product's host quantizer."""
    from slimkernels_amd import workloads
    z, names = _cases()
    for i, name in enumerate(names):
        d, M, N, K, g, mode, bf16 = _get(z, name)
        assert d["packed"].shape == (N, K // 4) and d["scales"].shape == (K // g, N)
        assert d["zp"].max() <= 3
        if mode == "sym":
            assert (d["zp"] == 2).all()
        if mode == "ref":
            assert (d["zp"] == 1).all()


@pytest.mark.gpu
@pytest.mark.parametrize("kernel", ["skinny", "tiled"])
def test_kernels_reproduce_golden(gpu_ops, kernel):
    import torch
    z, names = _cases()
    for name in names:
        d, M, N, K, g, mode, bf16 = _get(z, name)
        print("golden", name, kernel, flush=True)
        uniform = {"sym": 2, "ref": 1}.get(mode)
        w = gpu_ops.repack_w2(d["packed"], d["scales"].view(np.float16), None if uniform is not None else d["zp"], g,
                              zp_const=uniform if uniform is not None else 0)
        x = torch.from_numpy(d["x"].view(np.float16).copy()).cuda()
        qa = gpu_ops.quantize_act_int8(x, g)
        odt = torch.bfloat16 if bf16 else torch.float16
        out, acc = gpu_ops.w2a8_gemm(qa, w, odt, kernel=kernel, split_k=1, dump="groups")
        out2 = gpu_ops.w2a8_gemm(qa, w, odt, kernel=kernel, split_k=1)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(qa.q.cpu().numpy(), d["q"])
        np.testing.assert_array_equal(qa.s_a.cpu().numpy(), d["s_a"])
        np.testing.assert_array_equal(qa.rowsum.cpu().numpy()[:, :M], d["rowsum"])
        np.testing.assert_array_equal(acc.cpu().numpy(), d["acc"])
        for o in (out, out2):
            bits = o.view(torch.int16).cpu().numpy().view(np.uint16)
            if kernel == "tiled":
                np.testing.assert_array_equal(bits, d["out_bits"])
            else:  # K is one or two chunks here: the in-workgroup sum only reorders a handful of terms
                a = (bits.astype(np.uint32) << 16).view(np.float32) if bf16 else bits.view(np.float16).astype(np.float32)
                b = (d["out_bits"].astype(np.uint32) << 16).view(np.float32) if bf16 else d["out_bits"].view(np.float16).astype(np.float32)
                np.testing.assert_allclose(a, b, rtol=1e-3, atol=2.0 ** -24)
