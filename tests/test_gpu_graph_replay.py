"""Every entry point of the hot path recorded into one HIP graph and replayed: each replay, with eager work and
synchronisations between the replays, leaves the bits of the eager calls.  (The throughput figures are taken on graph
replays; split-K arrival counters and the fused form's row flags have to come back to zero inside the kernels for a
replay to be a repeat.)"""
import numpy as np
import pytest
import torch

from slimkernels_amd import _lib, workloads
import parity_utils as pu

pytestmark = pytest.mark.gpu


def _prepare(gpu_ops, M, N, K, g, mode, seed):
    case = pu.small_case(M, N, K, g, mode, seed=seed)
    packed, scales, zero = pu.quantized_weight(case)
    x = workloads.make_activation(case)
    w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
    return case, w, xd


def test_replays_repeat_the_eager_calls(gpu_ops):
    L = _lib.lib()
    # (M, N, K, group, mode, kernel): K split across workgroups wherever the library's own choice says so
    singles = [
        (16, 1024, 14336, 128, "sym", "skinny"),     # split-K through the workspace, counters reset in the kernel
        (24, 8192, 12288, 128, "asym", "skinny"),    # shared-activation workgroups, two row blocks, split-K
        (100, 1000, 12288, 128, "sym", "auto"),      # 33..256 rows
        (64, 4096, 4096, 128, "sym", "tiled"),       # tiled split-K
        (300, 520, 1024, 64, "ref", "tiled"),        # tiled, unsplit, zero-point prologue
        (80, 2048, 8192, 128, "asym", "mid"),        # the 33..128-row kernel, split-K (counters reset in the kernel)
    ]
    prepared = []
    for i, (M, N, K, g, mode, kernel) in enumerate(singles):
        case, w, xd = _prepare(gpu_ops, M, N, K, g, mode, 900 + i)
        prepared.append((case, w, xd, kernel, torch.empty((M, N), dtype=torch.float16, device="cuda")))
    assert L.slimk_w2a8_gemm_auto_split_k(16, 1024, 14336, 128, _lib.KERNEL_SKINNY) > 1
    assert L.slimk_w2a8_gemm_auto_split_k(64, 4096, 4096, 128, _lib.KERNEL_TILED) > 1
    assert L.slimk_w2a8_gemm_auto_split_k(80, 2048, 8192, 128, _lib.KERNEL_MID) > 1
    grouped = []
    for i, (M, N, K) in enumerate([(1, 2048, 4096), (16, 520, 2048), (32, 1024, 8192)]):
        case, w, xd = _prepare(gpu_ops, M, N, K, 128, "sym", 950 + i)
        grouped.append((case, w, xd, torch.empty((M, N), dtype=torch.float16, device="cuda")))
    fused = []
    for i, (M, N, K) in enumerate([(1, 2048, 4096), (8, 1024, 8192)]):   # in the workgroup / by the grid's first workgroups
        case, w, xd = _prepare(gpu_ops, M, N, K, 128, "sym", 970 + i)
        fused.append((case, w, xd))

    a16_xb = fused[0][2].to(torch.bfloat16)
    a16_outs = [torch.empty((1, 2048), dtype=torch.float16, device="cuda") for _ in range(2)] + \
               [torch.empty((c[0].M, c[0].N), dtype=torch.float16, device="cuda") for c in grouped]
    qas = {}
    static_outs = [torch.empty((p[0].M, p[0].N), dtype=torch.float16, device="cuda") for p in prepared[:1] + prepared[3:4]]

    def step():
        """act-quant + GEMM through every form; returns the outputs in a fixed order."""
        outs = []
        for case, w, xd, kernel, out in prepared:
            qa = gpu_ops.quantize_act_int8(xd, w.group_size)
            qas[case.name] = qa  # (keeps the buffers of the captured calls alive)
            outs.append(gpu_ops.w2a8_gemm(qa, w, torch.float16, kernel=kernel, out=out))
        probs = []
        for case, w, xd, out in grouped:
            qa = gpu_ops.quantize_act_int8(xd, w.group_size)
            qas[case.name] = qa
            probs.append((qa, w, out))
        outs += gpu_ops.w2a8_gemm_grouped(probs, torch.float16)
        for case, w, xd in fused:
            outs.append(gpu_ops.w2a8_linear_fused(xd, w, torch.float16))
        # the weight-only form: one launch with K split through its own partial-sum buffer, bf16 activations, and the
        # grouped launch
        case, w, xd = fused[0][0], fused[0][1], fused[0][2]
        outs.append(gpu_ops.w2a16_gemm(xd, w, torch.float16, split_k=2, out=a16_outs[0]))
        outs.append(gpu_ops.w2a16_gemm(a16_xb, w, torch.float16, out=a16_outs[1]))
        outs += gpu_ops.w2a16_gemm_grouped([(c[2], c[1], o) for c, o in zip(grouped, a16_outs[2:])], torch.float16)
        # the entry point that allocates nothing (split-K through the library-owned array): its first call on the
        # device is the eager one below, outside the capture
        for (case, w, xd, kernel, _), out in zip(prepared[:1] + prepared[3:4], static_outs):
            qa = qas[case.name]
            _lib.check(L.slimk_w2a8_gemm_static(
                qa.q.data_ptr(), qa.q.stride(0), qa.s_a.data_ptr(), qa.rowsum.data_ptr(), qa.rowsum.stride(0),
                w.w_r.data_ptr(), w.s_r.data_ptr(), None, w.zp_const, case.M, w.N, w.K, w.group_size,
                out.data_ptr(), out.stride(0), _lib.F16, {"skinny": _lib.KERNEL_SKINNY, "tiled": _lib.KERNEL_TILED}[kernel], 0,
                torch.cuda.current_stream().cuda_stream))
            outs.append(out)
        return outs

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):      # eagerly on the capturing stream first: its workspaces come to exist here
        want = [pu.out_tensor_bits(o) for o in step()]
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        outs = step()
    torch.cuda.synchronize()
    scratch = torch.empty(1 << 20, device="cuda")
    for replay in range(4):
        print("graph replay", replay, flush=True)
        for o in outs:
            o.zero_()
        scratch.normal_()                # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for o, w_bits in zip(outs, want):
            np.testing.assert_array_equal(pu.out_tensor_bits(o), w_bits, err_msg=f"replay {replay}")
