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
        kernel = rng.choice(["auto", "auto", "skinny", "tiled"])
        if kernel == "skinny" and case.M > 32:
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
