"""Seeded random shapes, level sets, output types, kernels and split-K values against the oracle: the same
criteria as the fixed cases (int8 activations and int32 group sums bit-exact, outputs within the tolerance
written in parity_utils.assert_out_close), on shapes nobody picked by hand -- ragged M and N around the
kernels' tile and policy boundaries, every group size, short and long reductions."""
import random

import numpy as np
import pytest
import torch

from slimkernels_amd import workloads
import parity_utils as pu

pytestmark = pytest.mark.gpu


def _random_case(rng, max_m):
    g = rng.choice([64, 128, 128, 256])
    K = g * rng.choice([1, 2, 3, 4, 6, 8, 13, 16, 24, 32, 56])
    M = rng.choice([m for m in (1, 1, 2, 3, 4, 5, 8, 13, 16, 17, 24, 31, 32, 33, 48, 64, 65, 77, 100, 128, 130, 200, 256, 300) if m <= max_m])
    N = rng.choice([1, 8, 63, 64, 65, 100, 128, 200, 256, 320, 512, 1000, 1024, 2048, 3000, 4096])
    while M * N * K > 2e8:
        if N > 64:
            N //= 2
        else:
            M = max(1, M // 2)
    mode = rng.choice(["sym", "sym", "asym", "ref"])
    odt = rng.choice(["float16", "bfloat16"])
    return pu.small_case(M, N, K, g, mode, seed=rng.randrange(1 << 20), out_dtype=odt, outliers=rng.random() < 0.3)


@pytest.mark.parametrize("seed", range(6))
def test_random_single_gemms(gpu_ops, oracle, seed):
    rng = random.Random(1000 + seed)
    checked = 0
    for _ in range(25):
        case = _random_case(rng, 300)
        kernel = rng.choice(["auto", "auto", "skinny", "tiled", "mid"])
        if kernel == "skinny" and case.M > 32:
            kernel = "auto"
        if kernel == "mid" and case.M > 256:
            kernel = "auto"
        split = 0 if rng.random() < 0.5 else rng.randint(1, 8)
        tag = f"M={case.M} N={case.N} K={case.K} g={case.group_size} {case.mode} {case.out_dtype} {kernel} split={split}"
        print(tag, flush=True)
        packed, scales, zero = workloads.make_quantized_weight(case)
        x = workloads.make_activation(case)
        bf16 = case.out_dtype == "bfloat16"
        ref = oracle.reference_forward(x, packed, scales, zero, case.group_size, out_bf16=bf16, want_acc=True)
        w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
        qa = gpu_ops.quantize_act_int8(xd, case.group_size)
        try:
            out, acc = gpu_ops.w2a8_gemm(qa, w, pu.torch_dtype(case), kernel=kernel, split_k=split, dump="groups")
            out2 = gpu_ops.w2a8_gemm(qa, w, pu.torch_dtype(case), kernel=kernel, split_k=split)
        except RuntimeError as e:          # a split-K value this shape and kernel do not take: a clean refusal
            assert split > 1 and "split" in str(e), f"{tag}: {e}"
            continue
        torch.cuda.synchronize()
        np.testing.assert_array_equal(qa.q.cpu().numpy(), ref["q"])
        np.testing.assert_array_equal(acc.cpu().numpy(), ref["acc"])
        bound = pu.reorder_bound(ref["acc"], scales, ref["s_a"])
        for o in (out, out2):
            pu.assert_out_close(pu.out_tensor_bits(o), ref["out_bits"], bf16, bound, tag)
        if case.M <= 32:
            o3 = gpu_ops.w2a8_linear_fused(xd, w, pu.torch_dtype(case))
            pu.assert_out_close(pu.out_tensor_bits(o3), ref["out_bits"], bf16, bound, tag + " fused")
        checked += 1
    assert checked >= 10


@pytest.mark.parametrize("seed", range(4))
def test_random_grouped_launches(gpu_ops, oracle, seed):
    rng = random.Random(2000 + seed)
    for _ in range(6):
        g = rng.choice([64, 128, 256])
        asym = rng.random() < 0.3
        odt = rng.choice(["float16", "bfloat16"])
        probs, refs, tags = [], [], []
        for _ in range(rng.randint(1, 8)):
            K = g * rng.choice([1, 2, 4, 8, 16, 32, 56])
            M = rng.choice([1, 2, 3, 4, 7, 8, 9, 15, 16, 17, 25, 32])
            N = rng.choice([8, 64, 65, 100, 256, 512, 1000, 2048, 4096])
            while M * N * K > 1e8:
                N = max(8, N // 2)
            mode = "asym" if asym else rng.choice(["sym", "ref"])
            case = pu.small_case(M, N, K, g, mode, seed=rng.randrange(1 << 20), out_dtype=odt)
            packed, scales, zero = workloads.make_quantized_weight(case)
            x = workloads.make_activation(case)
            ref = oracle.reference_forward(x, packed, scales, zero, g, out_bf16=odt == "bfloat16", want_acc=True)
            w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
            out = torch.empty((M, N), dtype=pu.torch_dtype(case), device="cuda")
            probs.append((gpu_ops.quantize_act_int8(xd, g), w, out))
            refs.append((ref, scales))
            tags.append(f"M={M} N={N} K={K} {mode}")
        print(f"grouped g={g} {odt}", tags, flush=True)
        gpu_ops.w2a8_gemm_grouped(probs, torch.bfloat16 if odt == "bfloat16" else torch.float16)
        torch.cuda.synchronize()
        for (_, _, out), (ref, scales), tag in zip(probs, refs, tags):
            pu.assert_out_close(pu.out_tensor_bits(out), ref["out_bits"], odt == "bfloat16",
                                pu.reorder_bound(ref["acc"], scales, ref["s_a"]), tag)


def _blas_reference(oracle, x, packed, scales, zero, g, bf16):
    """The oracle's forward with the int32 group sums formed by its exact float BLAS product (every partial sum is an
    integer below 2^24): the same numbers as reference_forward, in a time that allows every row of a chip-filling
    problem to be checked."""
    q, s_a, _ = oracle.c_act_quant(x, g)
    acc = oracle.np_gemm_acc_blas(q, oracle.np_unpack(packed), zero, g, dtype=np.float32)
    out_bits, _ = oracle.c_epilogue(acc, scales, s_a, bf16)
    return dict(q=q, s_a=s_a, acc=acc, out_bits=out_bits)


@pytest.mark.parametrize("seed", range(2))
def test_random_split_k_launches_of_more_workgroups_than_run_at_once(gpu_ops, oracle, seed):
    """Split-K of the tiled kernel (W2 and the one-pass W4 form) and of the kernel for 33..256 rows on launches of 600
    workgroups and more, one or two stages (rounds) per workgroup: the last workgroups to start publish their partial
    sums into a memory pipeline that is backed up.  Every output of every row against the oracle (not against the verification instantiation)."""
    from slimkernels_amd import w4
    from slimkernels_amd.torch import w4 as tw4
    rng = random.Random(3000 + seed)
    for it in range(3):
        g = rng.choice([64, 128, 256])
        split = rng.choice([4, 5, 6, 8])
        per = rng.choice([1, 2]) * (2 if g == 256 else 1)          # stages of 128 elements per split (whole groups of 256)
        K = 128 * per * split
        mt = rng.choice([3, 4])                                    # 64-row token tiles
        M = 64 * mt - rng.choice([0, 1, 30, 62])
        nt = -(-(600 + rng.randrange(300)) // (mt * split))        # 256-channel tiles: 600..900 workgroups
        N = 256 * nt - rng.choice([0, 8, 64, 200])
        mode = rng.choice(["sym", "sym", "asym"])
        odt = rng.choice(["float16", "bfloat16"])
        bf16 = odt == "bfloat16"
        case = pu.small_case(M, N, K, g, mode, seed=rng.randrange(1 << 20), out_dtype=odt)
        tag = f"M={M} N={N} K={K} g={g} {mode} {odt} tiled split={split} workgroups={mt * nt * split}"
        print(tag, flush=True)
        packed, scales, zero = workloads.make_quantized_weight(case)
        x = workloads.make_activation(case)
        ref = _blas_reference(oracle, x, packed, scales, zero, g, bf16)
        w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
        qa = gpu_ops.quantize_act_int8(xd, g)
        out = gpu_ops.w2a8_gemm(qa, w, pu.torch_dtype(case), kernel="tiled", split_k=split)
        out2 = gpu_ops.w2a8_gemm(qa, w, pu.torch_dtype(case), kernel="tiled", split_k=split)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(qa.q.cpu().numpy(), ref["q"])
        np.testing.assert_array_equal(pu.out_tensor_bits(out), pu.out_tensor_bits(out2))
        pu.assert_out_close(pu.out_tensor_bits(out), ref["out_bits"], bf16, pu.reorder_bound(ref["acc"], scales, ref["s_a"]), tag)
        del w, qa, out, out2
        # a launch of the same class through the kernel for 33..256 rows (its partial tiles leave as 16-byte stores too):
        # four strips x one row part per workgroup, one or two rounds of four pieces per split
        msplit = rng.choice([4, 8])
        mM = rng.choice([40, 77, 100, 150])
        parts = ((mM + 15) // 16 + 5) // 6
        mK = 64 * 4 * (1 if g == 64 else 2) * rng.choice([1, 2]) * msplit
        sets = -(-(600 + rng.randrange(300)) // (parts * msplit))
        mN = 256 * sets - rng.choice([0, 8, 64, 200])
        mcase = pu.small_case(mM, mN, mK, g, mode, seed=rng.randrange(1 << 20), out_dtype=odt)
        mtag = f"M={mM} N={mN} K={mK} g={g} {mode} {odt} mid split={msplit} workgroups={sets * parts * msplit}"
        print(mtag, flush=True)
        mpacked, mscales, mzero = workloads.make_quantized_weight(mcase)
        mx = workloads.make_activation(mcase)
        mref = _blas_reference(oracle, mx, mpacked, mscales, mzero, g, bf16)
        mw, mxd = pu.device_inputs(gpu_ops, mcase, mpacked, mscales, mzero, mx)
        mqa = gpu_ops.quantize_act_int8(mxd, g)
        mout = gpu_ops.w2a8_gemm(mqa, mw, pu.torch_dtype(mcase), kernel="mid", split_k=msplit)
        mout2 = gpu_ops.w2a8_gemm(mqa, mw, pu.torch_dtype(mcase), kernel="mid", split_k=msplit)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(pu.out_tensor_bits(mout), pu.out_tensor_bits(mout2))
        pu.assert_out_close(pu.out_tensor_bits(mout), mref["out_bits"], bf16, pu.reorder_bound(mref["acc"], mscales, mref["s_a"]), mtag)
        del mw, mqa, mout, mout2
        if g == 256:
            continue
        # the same launch shape through the one-pass 4-bit form of the body (uniform zero-point 8)
        rngw = np.random.default_rng(rng.randrange(1 << 20))
        w4f = (rngw.standard_normal((N, K), dtype=np.float32) * np.float32(0.02)).astype(np.float16).astype(np.float32)
        packed4, scales4, zp4 = w4.prepare_w4(w4f, g, "sym")
        ref4 = oracle.w4_reference_forward(x, w4.unpack_w4(packed4), scales4, zp4, g, out_bf16=bf16)
        w4d = tw4.repack_w4(packed4, scales4, zp4, g)
        qa = gpu_ops.quantize_act_int8(xd, g)
        print(tag.replace("tiled", "W4 one pass"), flush=True)
        y = tw4.w4a8_gemm_one_pass(qa, w4d, pu.torch_dtype(case), split_k=split)
        torch.cuda.synchronize()
        pu.assert_out_close(pu.out_tensor_bits(y), ref4["out_bits"], bf16, pu.reorder_bound(ref4["acc"], scales4, ref4["s_a"]),
                            tag + " W4 one pass")


@pytest.mark.parametrize("M,N,K,g,mode,odt", [
    (40, 8192, 12288, 64, "sym", "bfloat16"),      # 24 MiB: three row blocks
    (72, 8192, 16384, 128, "asym", "float16"),     # 32 MiB: five row blocks, per-group zero-points
    (33, 12352, 12288, 256, "ref", "float16"),     # ragged last strip set, groups of 256, one row in the third block
    (150, 8192, 16384, 128, "sym", "bfloat16"),    # two row parts of five blocks
])
def test_auto_takes_the_kernel_for_33_to_128_rows_on_large_matrices(gpu_ops, oracle, M, N, K, g, mode, odt):
    """Row counts that leave 64-row tiles partly empty, on large matrices, go to SLIMK_KERNEL_MID on the library's own
    choice (should the choice move, pick cases that it still sends there): every output of every row against the oracle (int32 sums by its exact float product), the int32 sums
    over K bit for bit, verification and production bits equal."""
    from slimkernels_amd import _lib
    assert _lib.lib().slimk_w2a8_gemm_auto_route(M, N, K, g) == 4
    bf16 = odt == "bfloat16"
    case = pu.small_case(M, N, K, g, mode, seed=M + N + K, out_dtype=odt)
    print(case.name, flush=True)
    packed, scales, zero = workloads.make_quantized_weight(case)
    x = workloads.make_activation(case)
    ref = _blas_reference(oracle, x, packed, scales, zero, g, bf16)
    w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
    qa = gpu_ops.quantize_act_int8(xd, g)
    out, acc = gpu_ops.w2a8_gemm(qa, w, pu.torch_dtype(case), kernel="auto", dump="sum")
    out2 = gpu_ops.w2a8_gemm(qa, w, pu.torch_dtype(case), kernel="auto")
    torch.cuda.synchronize()
    np.testing.assert_array_equal(qa.q.cpu().numpy(), ref["q"])
    np.testing.assert_array_equal(acc.cpu().numpy(), ref["acc"].sum(axis=2).astype(np.int64))
    np.testing.assert_array_equal(pu.out_tensor_bits(out), pu.out_tensor_bits(out2))
    pu.assert_out_close(pu.out_tensor_bits(out), ref["out_bits"], bf16, pu.reorder_bound(ref["acc"], scales, ref["s_a"]), case.name)
