"""slimk_w2a8_gemm_static, the GEMM entry point that allocates nothing (its split-K counters and partial sums live
in a device array inside the library), called through the C ABI and held bit for bit to slimk_w2a8_gemm with a
caller-owned workspace: calls in a row on one stream, each smaller than the one before, on every kernel that splits K."""
import numpy as np
import pytest
import torch

from slimkernels_amd import _lib, workloads
import parity_utils as pu

pytestmark = pytest.mark.gpu


def _call_static(L, qa, w, out, kernel, split_k):
    return L.slimk_w2a8_gemm_static(
        qa.q.data_ptr(), qa.q.stride(0), qa.s_a.data_ptr(), qa.rowsum.data_ptr(), qa.rowsum.stride(0),
        w.w_r.data_ptr(), w.s_r.data_ptr(), w.zp_r.data_ptr() if w.zp_r is not None else None, w.zp_const,
        qa.q.shape[0], w.N, w.K, w.group_size, out.data_ptr(), out.stride(0), _lib.F16,
        kernel, split_k, torch.cuda.current_stream().cuda_stream)


# (M, N, K, group, mode, kernel): every one splits K by the library's own choice; each call is smaller than the last
SEQUENCE = [
    (16, 4096, 14336, 128, "sym", _lib.KERNEL_SKINNY),
    (8, 2048, 14336, 128, "asym", _lib.KERNEL_SKINNY),
    (80, 2048, 8192, 128, "asym", _lib.KERNEL_MID),
    (64, 4096, 4096, 128, "sym", _lib.KERNEL_TILED),
    (40, 512, 8192, 64, "sym", _lib.KERNEL_TILED),
    (1, 2048, 14336, 128, "sym", _lib.KERNEL_SKINNY),
]


def test_gemm_without_allocation_matches_the_workspace_entry_point(gpu_ops, oracle):
    L = _lib.lib()
    assert L.slimk_w2a8_static_workspace_bytes() == (16 << 20) + (64 << 10)
    prepared = []
    for i, (M, N, K, g, mode, kernel) in enumerate(SEQUENCE):
        case = pu.small_case(M, N, K, g, mode, seed=400 + i)
        packed, scales, zero = pu.quantized_weight(case)
        x = workloads.make_activation(case)
        w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
        qa = gpu_ops.quantize_act_int8(xd, g)
        kname = {_lib.KERNEL_SKINNY: "skinny", _lib.KERNEL_TILED: "tiled", _lib.KERNEL_MID: "mid"}[kernel]
        assert L.slimk_w2a8_gemm_auto_split_k(M, N, K, g, kernel) > 1, "the case is meant to split K"
        want = gpu_ops.w2a8_gemm(qa, w, torch.float16, kernel=kname)      # caller-owned workspace
        ref = oracle.reference_forward(x, packed, scales, zero, g, want_acc=True)
        prepared.append((case, qa, w, want, ref, scales, kernel))
    torch.cuda.synchronize()
    outs = [torch.empty_like(p[3]) for p in prepared]
    held = torch.cuda.memory_allocated()
    for rnd in range(2):                                                 # the whole sequence twice, back to back
        for (case, qa, w, want, ref, scales, kernel), out in zip(prepared, outs):
            print("gemm_static", case.name, "round", rnd, flush=True)
            out.zero_()
            _lib.check(_call_static(L, qa, w, out, kernel, 0))
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == held
        for (case, qa, w, want, ref, scales, kernel), out in zip(prepared, outs):
            np.testing.assert_array_equal(pu.out_tensor_bits(out), pu.out_tensor_bits(want), err_msg=case.name)
            pu.assert_out_close(pu.out_tensor_bits(out), ref["out_bits"], False,
                                pu.reorder_bound(ref["acc"], scales, ref["s_a"]), "gemm_static " + case.name)


def test_gemm_without_allocation_rejects_what_does_not_fit(gpu_ops):
    L = _lib.lib()
    case = pu.small_case(512, 4096, 14336, 128, "sym", seed=7)
    packed, scales, zero = pu.quantized_weight(case)
    w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, workloads.make_activation(case))
    qa = gpu_ops.quantize_act_int8(xd, 128)
    out = torch.empty((512, 4096), dtype=torch.float16, device="cuda")
    # eight splits of 128 tiles of 64 x 256 fp32: 64 MiB of partial sums
    assert L.slimk_w2a8_gemm_workspace_bytes(512, 4096, 14336, 128, _lib.KERNEL_TILED, 8) > L.slimk_w2a8_static_workspace_bytes()
    rc = _call_static(L, qa, w, out, _lib.KERNEL_TILED, 8)
    assert rc == 5 and b"library-owned" in L.slimk_w2a8_last_error()
    # left to the library, the split is lowered until it fits; the result is that split's through the other entry point
    _lib.check(_call_static(L, qa, w, out, _lib.KERNEL_TILED, 0))
    fit = 8
    while L.slimk_w2a8_gemm_workspace_bytes(512, 4096, 14336, 128, _lib.KERNEL_TILED, fit) > L.slimk_w2a8_static_workspace_bytes():
        fit -= 1
    fit = min(fit, L.slimk_w2a8_gemm_auto_split_k(512, 4096, 14336, 128, _lib.KERNEL_TILED))
    want = gpu_ops.w2a8_gemm(qa, w, torch.float16, kernel="tiled", split_k=fit)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(pu.out_tensor_bits(out), pu.out_tensor_bits(want))
