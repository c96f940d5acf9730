"""GPU parity: the HIP kernels (through the C ABI) against the CPU oracle on the same seeded
inputs.  int8 / int32 / index results must be bit-exact; fp16 / bf16 outputs within
rtol 1e-3 or 1 ULP of the output type (the tiled kernel, which sums groups in the oracle's
order with the same fused multiply-add, is additionally required to be bit-identical)."""
import numpy as np
import pytest
import torch

from slimkernels_amd import layout, workloads
import parity_utils as pu

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


# ------------------------------------------------------------------ repack
@pytest.mark.parametrize("N,K,g,with_zp", [(64, 64, 64, False), (100, 256, 128, True), (4096, 4096, 128, False),
                                           (1000, 512, 256, True), (16, 128, 64, True), (130, 576, 64, True),
                                           (77, 1408, 128, False)])
def test_repack_matches_layout_definition(gpu_ops, N, K, g, with_zp):
    _say("repack", N, K, g, with_zp)
    rng = np.random.default_rng(N + K)
    packed = rng.integers(0, 256, (N, K // 4), dtype=np.uint8)
    scales = rng.uniform(0.001, 0.03, (K // g, N)).astype(np.float16)
    zp = rng.integers(0, 4, (K // g, N), dtype=np.uint8) if with_zp else None
    w = gpu_ops.repack_w2(packed, scales, zp, g)
    strips, steps = -(-N // 64), K // 64
    got = w.w_r.cpu().numpy().view(np.uint32).reshape(-(-steps // 4), strips, 4, 64, 4)
    np.testing.assert_array_equal(got, layout.repack_codes(packed))
    np.testing.assert_array_equal(layout.unrepack_codes(got, N, K), packed)
    np.testing.assert_array_equal(w.s_r.cpu().numpy().reshape(K // g, strips, 16, 4), layout.repack_group_values(scales))
    if with_zp:
        np.testing.assert_array_equal(w.zp_r.cpu().numpy().reshape(K // g, strips, 16, 4), layout.repack_group_values(zp))


# ------------------------------------------------------------------ weight quantisation on the GPU
@pytest.mark.parametrize("N,K,g,mode,bf16", [(64, 256, 128, "sym", False), (100, 512, 64, "asym", False),
                                             (7, 768, 256, "ref", False), (130, 1024, 128, "asym", True),
                                             (33, 8192, 128, "sym", True), (256, 4096, 64, "ref", False)])
def test_weight_quantisation_on_gpu_bit_exact(gpu_ops, oracle, N, K, g, mode, bf16):
    """fp16 / bf16 weight -> packed codes, fp16 scales, zero-points: the host functions' numbers."""
    from slimkernels_amd import prepare_w2
    _say("quantize_weight", N, K, g, mode, bf16)
    rng = np.random.default_rng(N + K)
    w = rng.normal(0, 0.02, (N, K)).astype(np.float32)
    w[0, :g] = 0.0                                   # an all-zero group: scale floor, codes = zero-point
    w[min(1, N - 1), 3] = 0.5                        # an outlier that sets its group's scale
    wt = torch.from_numpy(w).to(torch.bfloat16 if bf16 else torch.float16)
    # ties: values at exactly (level + 0.5) * scale of their group (scale = absmax / 2 resp. / 1.5)
    if mode != "asym":
        div = 2.0 if mode == "sym" else 1.5
        wt[min(2, N - 1), :g] = 0.0
        wt[min(2, N - 1), 0] = 1.0
        for i, lv in enumerate((0.5, -0.5, 1.5, -1.5, 2.5, -2.5)):
            wt[min(2, N - 1), 1 + i] = lv / div
    host = prepare_w2(wt.float().numpy(), g, mode)
    packed, scales, zero = gpu_ops.quantize_weight_gpu(wt.cuda(), g, mode)
    torch.cuda.synchronize()
    # against the oracle itself: its C quantiser on the [K, N] matrix, its packer on the transposed codes, its
    # float32 scales rounded once to float16
    o_codes, o_scales, o_zp = oracle.c_quantize_w2(np.ascontiguousarray(wt.float().numpy().T), g, mode)
    np.testing.assert_array_equal(packed.cpu().numpy(), oracle.c_pack(np.ascontiguousarray(o_codes.T)))
    np.testing.assert_array_equal(scales.cpu().numpy().view(np.uint16), o_scales.astype(np.float16).view(np.uint16))
    np.testing.assert_array_equal(zero.cpu().numpy(), o_zp)
    # and against the package's host functions
    np.testing.assert_array_equal(packed.cpu().numpy(), host[0])
    np.testing.assert_array_equal(scales.cpu().numpy().view(np.uint16), host[1].view(np.uint16))
    np.testing.assert_array_equal(zero.cpu().numpy(), host[2])
    # a strided view (rows of a wider matrix) takes the same path
    wide = torch.zeros(N, K + 8, dtype=wt.dtype, device="cuda")
    wide[:, :K] = wt.cuda()
    packed2, scales2, zero2 = gpu_ops.quantize_weight_gpu(wide[:, :K], g, mode)
    assert torch.equal(packed, packed2) and torch.equal(scales, scales2) and torch.equal(zero, zero2)
    # and the layer built from the device tensor equals the one built on the host
    lin_d = gpu_ops.W2A8Linear.from_float(wt.cuda(), g, mode)
    lin_h = gpu_ops.W2A8Linear.from_float(wt.float().numpy(), g, mode)
    assert torch.equal(lin_d.weight.w_r, lin_h.weight.w_r) and torch.equal(lin_d.weight.s_r, lin_h.weight.s_r)


# ------------------------------------------------------------------ activation quantisation
@pytest.mark.parametrize("M,K,g,bf16,outliers", [(1, 4096, 128, False, True), (16, 4096, 128, False, True),
                                                 (77, 4096, 128, False, False), (3, 13824, 128, False, False),
                                                 (5, 8192, 64, True, False), (33, 256, 256, False, False),
                                                 (2, 64, 64, False, False),
                                                 # many rows, long rows, odd row counts
                                                 (64, 4096, 128, False, True), (77, 8192, 64, True, False),
                                                 (130, 14336, 128, False, True), (67, 192, 64, False, False),
                                                 (65, 6144, 256, True, False), (66, 16448, 64, False, False),
                                                 # a few long rows: 1024 threads a row (one, two or four vectors each)
                                                 (16, 14336, 128, False, True), (64, 8192, 128, True, False),
                                                 (3, 28672, 64, False, False), (32, 32768, 256, False, False),
                                                 (7, 33280, 64, False, False)])
def test_act_quant_bit_exact(gpu_ops, oracle, M, K, g, bf16, outliers):
    _say("act_quant", M, K, g, bf16)
    case = pu.small_case(M, 64, K, g, "sym", seed=M * 7 + K, outliers=outliers)
    x = workloads.make_activation(case)
    x[min(1, M - 1), : min(K, 70)] = 0.0
    if M > 2:
        x[2] = 0.0  # an all-zero token
    if M > 4:
        # exact and near ties of the rounding: a row whose scale is exactly 1 (absmax 127) holding k + 1/2, and one whose
        # scale is a hair above 1, so that the same values land just below the tie points
        ties = (np.arange(K) % 253 - 126).astype(np.float32) + 0.5
        x[3] = ties.astype(np.float16)
        x[3, 0] = 127.0
        x[4] = ties.astype(np.float16)
        x[4, 0] = 127.0625
    if bf16:
        xt = torch.from_numpy(x.astype(np.float32)).to(torch.bfloat16)
        bits = xt.view(torch.int16).numpy().view(np.uint16)
        q, s_a, rs = oracle.c_act_quant(bits, g, is_bf16=True)
    else:
        xt = torch.from_numpy(x)
        q, s_a, rs = oracle.c_act_quant(x, g)
    qa = gpu_ops.quantize_act_int8(xt.cuda(), g)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(qa.s_a.cpu().numpy(), s_a)
    np.testing.assert_array_equal(qa.q.cpu().numpy(), q)
    np.testing.assert_array_equal(qa.rowsum.cpu().numpy()[:, :M], rs)


@pytest.mark.parametrize("M,K", [(8, 4096), (16, 8192), (3, 28672), (80, 4096), (70, 20480), (130, 14336)])
def test_act_quant_values_next_to_rounding_ties(gpu_ops, oracle, M, K):
    """Rows of values chosen next to the ties of q = rne(x / s): for a random absmax A (s = A / 127) the fp16 numbers
    nearest to (k + 1/2) * s and their neighbours.  The kernels round x * (1 / s) and fall back on the IEEE division
    near a tie (the forms for a few rows, for many rows, and the two-pass form for very long rows): all must give the
    oracle's bits."""
    _say("act_quant near ties", M, K)
    rng = np.random.default_rng(M * 31 + K)
    x = np.zeros((M, K), np.float16)
    for m in range(M):
        A = np.float16(rng.uniform(0.01, 300.0))
        s = np.float32(max(np.float32(A), np.float32(1e-9))) / np.float32(127.0)
        k = rng.integers(-127, 127, K).astype(np.float32) + 0.5
        base = (k * s).astype(np.float16)
        step = rng.integers(-2, 3, K)          # up to two fp16 neighbours either side
        moved = base.copy()
        for d in (1, 2):
            moved = np.where(step >= d, np.nextafter(moved, np.float16(np.inf)), moved)
            moved = np.where(step <= -d, np.nextafter(moved, np.float16(-np.inf)), moved)
        moved = np.clip(moved.astype(np.float32), -np.float32(A), np.float32(A)).astype(np.float16)
        moved[rng.integers(K)] = A              # the row's absmax is exactly A
        x[m] = moved
    q, s_a, rs = oracle.c_act_quant(x, 128)
    qa = gpu_ops.quantize_act_int8(torch.from_numpy(x).cuda(), 128)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(qa.s_a.cpu().numpy(), s_a)
    np.testing.assert_array_equal(qa.q.cpu().numpy(), q)
    np.testing.assert_array_equal(qa.rowsum.cpu().numpy()[:, :M], rs)


# ------------------------------------------------------------------ GEMM on small and ragged shapes
def _run_case(gpu_ops, oracle, case, kernel, split_k=0, dump="groups", exact_out=False, same_bits=True, strict=False):
    """One GEMM twice: with the int32 dump (the verification instantiation of the kernel body the call
    selects) and without (the production instantiation of the same body).  int8 activations and int32
    accumulators exact; outputs bit-identical with the oracle (exact_out), or within rtol 1e-3 / 1 ULP
    (strict: kernels that sum in the oracle's order), or additionally within the re-association bound."""
    _say("gemm", case.name, kernel, "split", split_k, "dump", dump)
    packed, scales, zero = pu.quantized_weight(case)
    x = workloads.make_activation(case)
    bf16 = case.out_dtype == "bfloat16"
    ref = oracle.reference_forward(x, packed, scales, zero, case.group_size, out_bf16=bf16, want_acc=True)
    w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
    qa = gpu_ops.quantize_act_int8(xd, case.group_size)
    out, acc = gpu_ops.w2a8_gemm(qa, w, pu.torch_dtype(case), kernel=kernel, split_k=split_k, dump=dump)
    out2 = gpu_ops.w2a8_gemm(qa, w, pu.torch_dtype(case), kernel=kernel, split_k=split_k)  # production instantiation
    torch.cuda.synchronize()
    np.testing.assert_array_equal(qa.q.cpu().numpy(), ref["q"])
    if dump == "groups":
        np.testing.assert_array_equal(acc.cpu().numpy(), ref["acc"])
    else:
        np.testing.assert_array_equal(acc.cpu().numpy(), ref["acc"].sum(axis=2))
    bound = pu.reorder_bound(ref["acc"], scales, ref["s_a"])
    for o in (out, out2):
        bits = pu.out_tensor_bits(o)
        if exact_out:
            np.testing.assert_array_equal(bits, ref["out_bits"])
        else:
            pu.assert_out_close(bits, ref["out_bits"], bf16, None if strict else bound, case.name)
    if same_bits:  # the verification instantiation and the production one are the same kernel body
        np.testing.assert_array_equal(pu.out_tensor_bits(out), pu.out_tensor_bits(out2))


SMALL = [
    # M, N, K, g, mode, out
    (1, 64, 128, 64, "sym", "float16"),
    (16, 128, 512, 128, "sym", "float16"),
    (7, 100, 256, 128, "asym", "float16"),
    (32, 192, 1024, 256, "sym", "bfloat16"),
    (17, 70, 768, 64, "asym", "bfloat16"),
    (3, 4096, 256, 128, "ref", "float16"),
]


@pytest.mark.parametrize("M,N,K,g,mode,out", SMALL)
def test_skinny_small(gpu_ops, oracle, M, N, K, g, mode, out):
    case = pu.small_case(M, N, K, g, mode, seed=M + N, out_dtype=out)
    _run_case(gpu_ops, oracle, case, "skinny", split_k=1)
    _run_case(gpu_ops, oracle, case, "skinny", split_k=0, dump="sum")
    G = K // g
    if G >= 2:
        _run_case(gpu_ops, oracle, case, "skinny", split_k=2)


@pytest.mark.parametrize("M,N,K,g,mode,out,split", [
    (16, 64, 8192, 128, "sym", "float16", 1),
    (16, 130, 8256, 64, "asym", "bfloat16", 1),   # 129 steps: the last pair of steps is half past the end
    (29, 70, 8320, 64, "sym", "float16", 1),      # two row blocks, the second ragged
    (32, 64, 9216, 256, "asym", "float16", 2),
    (20, 128, 8192, 128, "sym", "bfloat16", 3),
])
def test_skinny_wide_activation_fetch(gpu_ops, oracle, M, N, K, g, mode, out, split):
    """From 16 token rows and K >= 8192 on the skinny kernel fetches activations two steps wide and
    turns them through LDS: same results as the step-by-step fetch (int32 sums exact)."""
    case = pu.small_case(M, N, K, g, mode, seed=M + K, out_dtype=out)
    _run_case(gpu_ops, oracle, case, "skinny", split_k=split)
    _run_case(gpu_ops, oracle, case, "skinny", split_k=0, dump="sum")


@pytest.mark.parametrize("M,N,K,g,mode,out,split", [
    (33, 4096, 4096, 128, "sym", "float16", 0),     # the library's own choice for these rows and sizes
    (77, 200, 512, 128, "asym", "float16", 1),      # five row blocks, the last ragged
    (100, 130, 2048, 64, "sym", "bfloat16", 1),
    (256, 64, 1024, 256, "ref", "float16", 1),
    (64, 192, 4096, 128, "asym", "bfloat16", 1),    # eight waves per workgroup
    (48, 128, 14336, 128, "sym", "float16", 4),     # K split across workgroups: sixteen-wave workgroups
])
def test_skinny_more_than_32_rows(gpu_ops, oracle, M, N, K, g, mode, out, split):
    """33..256 token rows through the weight-streaming kernel (16 rows per workgroup and pass over the weights, the
    passes side by side): int32 sums exact, the output criterion, verification and production instantiation
    bit-identical."""
    case = pu.small_case(M, N, K, g, mode, seed=M + N + K, out_dtype=out)
    _run_case(gpu_ops, oracle, case, "skinny", split_k=split)
    _run_case(gpu_ops, oracle, case, "auto", split_k=0, dump="sum")


@pytest.mark.parametrize("M,N,K,g,mode,out,split", [
    (17, 6144, 16384, 128, "sym", "float16", 0),    # the second row block holds one row
    (20, 4096, 24576, 64, "asym", "bfloat16", 0),
    (25, 12352, 8192, 256, "sym", "float16", 3),    # ragged last strip set, explicit split
    (32, 8192, 12288, 128, "ref", "float16", 1),    # unsplit
])
def test_skinny_shared_one_problem(gpu_ops, oracle, M, N, K, g, mode, out, split):
    """17..32 token rows on a matrix of 24 MiB or more: one problem runs through the shared-activation
    workgroups with K split across workgroups; the int32 dump comes from the same body."""
    case = pu.small_case(M, N, K, g, mode, seed=M + K, out_dtype=out)
    _run_case(gpu_ops, oracle, case, "skinny", split_k=split, dump="sum")


@pytest.mark.parametrize("M,N,K,g,mode,out,split", [
    (14, 24640, 512, 64, "asym", "bfloat16", 0),    # two chunks for four k-parts: two of them idle
    (16, 24577, 2048, 128, "sym", "float16", 0),    # ragged last strip, odd number of two-strip units
    (12, 25000, 1280, 256, "ref", "float16", 2),    # explicit split, groups of 256
])
def test_skinny_shared_12_to_16_rows_on_wide_matrices(gpu_ops, oracle, M, N, K, g, mode, out, split):
    """12..16 token rows on 384 strips and more run through shared-activation workgroups of four k-parts x two
    strips: int32 group sums exact, the output criterion, verification and production bits equal."""
    from slimkernels_amd import _lib
    assert _lib.lib().slimk_w2a8_gemm_auto_route(M, N, K, g) == 3
    case = pu.small_case(M, N, K, g, mode, seed=M + N + K, out_dtype=out)
    _run_case(gpu_ops, oracle, case, "auto", split_k=split, dump="groups")
    _run_case(gpu_ops, oracle, case, "skinny", split_k=split)


@pytest.mark.parametrize("M,N,K,g,mode,out,split", [
    (100, 7400, 2304, 64, "asym", "bfloat16", 0),   # short reduction: seven row blocks, the last ragged, ragged last strip
    (130, 1000, 12288, 128, "sym", "float16", 0),   # long reduction, few strips: nine row blocks, K split across workgroups
    (33, 4000, 12288, 256, "ref", "float16", 0),    # the third row block holds one row
    (50, 4000, 12288, 128, "sym", "float16", 2),    # explicit split
    (250, 4000, 2304, 128, "asym", "float16", 0),   # sixteen row blocks
])
def test_skinny_shared_more_than_32_rows(gpu_ops, oracle, M, N, K, g, mode, out, split):
    """33..256 token rows where the library sends them through the shared-activation workgroups (one workgroup per
    four strips and block of 16 rows): int32 sums exact, the output criterion, and the library's own choice of kernel
    is that form (should the choice move, pick cases that it still sends there)."""
    from slimkernels_amd import _lib
    assert _lib.lib().slimk_w2a8_gemm_auto_route(M, N, K, g) == 3
    case = pu.small_case(M, N, K, g, mode, seed=M + N + K, out_dtype=out)
    _run_case(gpu_ops, oracle, case, "auto", split_k=split, dump="sum")
    _run_case(gpu_ops, oracle, case, "skinny", split_k=split)


@pytest.mark.parametrize("M,N,K,g,mode,out,split", [
    (33, 4000, 4096, 128, "sym", "float16", 0),      # three row blocks, the last with one row
    (77, 2752, 4096, 128, "asym", "float16", 0),     # five row blocks, per-group zero-points
    (128, 1000, 8192, 64, "sym", "bfloat16", 0),     # two row parts of four blocks, groups of 64
    (100, 520, 2560, 256, "ref", "float16", 2),      # row parts of four and three blocks, groups of 256 (two pieces each), one strip in the last set
    (64, 300, 1024, 64, "asym", "float16", 1),       # four row blocks, ragged last strip
    (90, 200, 1536, 128, "sym", "bfloat16", 3),      # six row blocks
    (48, 128, 192, 64, "sym", "float16", 1),         # three pieces: a round with a dead piece
    (40, 64, 256, 256, "ref", "float16", 1),         # a single group
    (20, 192, 2048, 128, "asym", "float16", 2),      # fewer rows than the form is meant for
    (112, 700, 2048, 128, "asym", "bfloat16", 0),    # seven row blocks: row parts of four and three
    (96, 1100, 3072, 256, "sym", "float16", 4),      # six row blocks, groups of 256, ragged last strip set
    (144, 600, 2048, 128, "sym", "float16", 2),      # nine row blocks: two row parts of five (the second holds four)
    (200, 320, 1024, 64, "asym", "bfloat16", 0),     # thirteen row blocks: three row parts of five (the third holds three)
])
def test_mid_kernel(gpu_ops, oracle, M, N, K, g, mode, out, split):
    """SLIMK_KERNEL_MID (a workgroup = four strips x up to six blocks of 16 token rows, the activations shared through
    LDS, K split across workgroups): int32 group sums exact, the output criterion, verification and production bits equal."""
    case = pu.small_case(M, N, K, g, mode, seed=M + N + K, out_dtype=out)
    _run_case(gpu_ops, oracle, case, "mid", split_k=split, dump="groups")
    _run_case(gpu_ops, oracle, case, "mid", split_k=split, dump="sum")


@pytest.mark.parametrize("M,N,K,g,mode,out", SMALL + [
    (77, 200, 512, 128, "asym", "float16"),
    (129, 130, 320, 64, "sym", "float16"),
    (300, 64, 256, 128, "sym", "bfloat16"),
    # groups of 256: a group spans two stages of the tiled kernel and its int32 sums stay in registers between them
    (70, 130, 2560, 256, "sym", "float16"),
    (100, 300, 1024, 256, "asym", "bfloat16"),
    (64, 256, 256, 256, "ref", "float16"),
    # an odd number of 64-element steps: the last stage's second step lies past the end of K
    (200, 256, 64, 64, "sym", "float16"),
    (77, 100, 448, 64, "asym", "float16"),
])
def test_tiled_small(gpu_ops, oracle, M, N, K, g, mode, out):
    case = pu.small_case(M, N, K, g, mode, seed=M + N + 1, out_dtype=out)
    # unsplit and with the zero-point the operand bytes are centred on (the symmetric levels), the tiled
    # kernels sum the groups in the oracle's order: bit-identical outputs.  Other zero-points add their
    # term through fp32 MFMAs first: the output criterion.
    exact = mode == "sym"
    _run_case(gpu_ops, oracle, case, "tiled", split_k=1, dump="groups", exact_out=exact)
    _run_case(gpu_ops, oracle, case, "tiled", split_k=1, dump="sum", exact_out=exact)
    # whatever split the library picks by itself (K may be split when tiles are few): the output criterion
    _run_case(gpu_ops, oracle, case, "tiled", split_k=0, dump="sum")


@pytest.mark.parametrize("M,N,K,g,out", [(70, 256, 512, 128, "float16"), (130, 320, 768, 64, "bfloat16")])
def test_tiled_output_views(gpu_ops, oracle, M, N, K, g, out):
    """The tiled kernel stores 16 bytes per lane when N, the row pitch and the address of out allow
    it and 2 bytes per value otherwise: a contiguous output, one that starts two bytes off a
    16-byte boundary and one with an odd row pitch hold the same bits."""
    _say("tiled output views", M, N, K, g, out)
    case = pu.small_case(M, N, K, g, "sym", seed=M + N + K, out_dtype=out)
    packed, scales, zero = pu.quantized_weight(case)
    x = workloads.make_activation(case)
    ref = oracle.reference_forward(x, packed, scales, zero, g, out_bf16=(out == "bfloat16"))
    w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
    qa = gpu_ops.quantize_act_int8(xd, g)
    odt = pu.torch_dtype(case)
    plain = gpu_ops.w2a8_gemm(qa, w, odt, kernel="tiled", split_k=1)
    wide = torch.zeros(M, N + 8, dtype=odt, device="cuda")
    odd = torch.zeros(M, N + 3, dtype=odt, device="cuda")
    shifted = gpu_ops.w2a8_gemm(qa, w, odt, kernel="tiled", split_k=1, out=wide[:, 1:1 + N])
    pitched = gpu_ops.w2a8_gemm(qa, w, odt, kernel="tiled", split_k=1, out=odd[:, :N])
    torch.cuda.synchronize()
    np.testing.assert_array_equal(pu.out_tensor_bits(plain), ref["out_bits"])
    np.testing.assert_array_equal(pu.out_tensor_bits(shifted.contiguous()), ref["out_bits"])
    np.testing.assert_array_equal(pu.out_tensor_bits(pitched.contiguous()), ref["out_bits"])
    assert float(wide[:, 0].abs().max()) == 0.0 and float(wide[:, 1 + N:].abs().max()) == 0.0
    assert float(odd[:, N:].abs().max()) == 0.0


@pytest.mark.parametrize("M,N,K,g,out,split", [(64, 256, 2048, 128, "float16", 2), (77, 300, 4096, 64, "bfloat16", 4),
                                                 (130, 64, 3072, 128, "float16", 3), (40, 512, 8192, 128, "float16", 8),
                                                 (64, 256, 4096, 256, "float16", 3), (77, 300, 4160, 64, "bfloat16", 4),
                                                 (50, 128, 2816, 256, "bfloat16", 11),
                                                 # more workgroups than run at once, one stage each: the last ones to start
                                                 # find the memory pipeline backed up when they store their partial sums
                                                 (130, 4096, 1024, 64, "bfloat16", 8), (130, 4096, 2048, 128, "float16", 8)])
def test_tiled_split_k(gpu_ops, oracle, M, N, K, g, out, split):
    """Split-K of the fast tiled kernel: the output criterion, and run-to-run identical bits."""
    case = pu.small_case(M, N, K, g, "sym", seed=M + K, out_dtype=out)
    packed, scales, zero = pu.quantized_weight(case)
    x = workloads.make_activation(case)
    bf16 = out == "bfloat16"
    w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
    qa = gpu_ops.quantize_act_int8(xd, g)
    outs = [pu.out_tensor_bits(gpu_ops.w2a8_gemm(qa, w, pu.torch_dtype(case), kernel="tiled", split_k=split)) for _ in range(4)]
    for o in outs[1:]:
        np.testing.assert_array_equal(o, outs[0])
    ref = oracle.reference_forward(x, packed, scales, zero, g, out_bf16=bf16)
    pu.assert_out_close(outs[0], ref["out_bits"], bf16, pu.reorder_bound(ref["acc"], scales, ref["s_a"]), f"tiled split {split}")


def test_split_k_is_deterministic_and_workspace_reusable(gpu_ops, oracle):
    case = pu.small_case(16, 256, 2048, 128, "sym", seed=5)
    packed, scales, zero = pu.quantized_weight(case)
    x = workloads.make_activation(case)
    w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
    qa = gpu_ops.quantize_act_int8(xd, 128)
    outs = [pu.out_tensor_bits(gpu_ops.w2a8_gemm(qa, w, kernel="skinny", split_k=4)) for _ in range(5)]
    for o in outs[1:]:
        np.testing.assert_array_equal(o, outs[0])
    ref = oracle.reference_forward(x, packed, scales, zero, 128)
    pu.assert_out_close(outs[0], ref["out_bits"], False, pu.reorder_bound(ref["acc"], scales, ref["s_a"]), "split4")


# ------------------------------------------------------------------ the configured workloads
def test_config_c1(gpu_ops, oracle):
    case = workloads.config_cases("c1")[0]
    _run_case(gpu_ops, oracle, case, "auto")
    _run_case(gpu_ops, oracle, case, "tiled", exact_out=True)


@pytest.mark.parametrize("shape", ["qo", "kv", "gate_up", "down"])
@pytest.mark.parametrize("M", list(workloads.DECODE_M))
def test_config_c2_decode(gpu_ops, oracle, shape, M):
    N, K = workloads.LLAMA8B_LINEARS[shape]
    case = workloads.Case("c2", M, N, K, outliers=True)
    _run_case(gpu_ops, oracle, case, "auto")


def test_config_c2_as_one_grouped_launch(gpu_ops, oracle):
    """The benchmark's step: exactly the 24 GEMMs of the decode sweep (M in {1,2,4,8,16,32} x the four Llama-3-8B
    linears, outlier channels) issued as ONE grouped launch.  The verification instantiation of the grouped kernel
    gives every problem's int32 accumulators (exact against the oracle); the production launch's outputs are
    bit-identical with the verification launch's and meet the output criterion against the oracle."""
    cases = workloads.config_cases("c2")
    assert len(cases) == 24
    weights, probs, refs = {}, [], []
    for c in cases:
        if (c.N, c.K) not in weights:
            packed, scales, zero = pu.quantized_weight(c)
            weights[(c.N, c.K)] = (packed, scales, zero, gpu_ops.repack_w2(packed, scales, None, c.group_size, zp_const=2))
        packed, scales, zero, w = weights[(c.N, c.K)]
        x = workloads.make_activation(c)
        probs.append((gpu_ops.quantize_act_int8(torch.from_numpy(x).cuda(), c.group_size), w))
        refs.append((oracle.reference_forward(x, packed, scales, zero, c.group_size, want_acc=True), scales))
    _say("grouped launch of the", len(probs), "c2 problems")
    outs = gpu_ops.w2a8_gemm_grouped(probs)
    outs_v, accs = gpu_ops.w2a8_gemm_grouped(probs, dump="groups")
    torch.cuda.synchronize()
    for c, o, ov, acc, (ref, scales) in zip(cases, outs, outs_v, accs, refs):
        np.testing.assert_array_equal(acc.cpu().numpy(), ref["acc"], err_msg=c.name)
        np.testing.assert_array_equal(pu.out_tensor_bits(o), pu.out_tensor_bits(ov), err_msg=c.name)
        pu.assert_out_close(pu.out_tensor_bits(o), ref["out_bits"], False,
                            pu.reorder_bound(ref["acc"], scales, ref["s_a"]), "c2 grouped " + c.name)


def test_workspace_serves_changing_shapes(gpu_ops, oracle):
    """One weight object, one lazily created split-K workspace, token counts that change from call to call (tiled
    split 8 -> skinny split 4, and two tiled splits with different tile counts): the arrival counters sit in a block
    of fixed size in front of the partial sums, so a later call's counters never land on an earlier call's partials."""
    N, K, g = 4096, 14336, 128
    base = pu.small_case(1, N, K, g, "sym", seed=21)
    packed, scales, zero = pu.quantized_weight(base)
    w = gpu_ops.repack_w2(packed, scales, None, g, zp_const=2)
    for M in (64, 20, 256, 320, 20, 64):
        case = pu.small_case(M, N, K, g, "sym", seed=100 + M)
        x = workloads.make_activation(case)
        ref = oracle.reference_forward(x, packed, scales, zero, g, want_acc=True)
        out = gpu_ops.w2a8_gemm(gpu_ops.quantize_act_int8(torch.from_numpy(x).cuda(), g), w)
        torch.cuda.synchronize()
        _say("workspace reuse M", M, "workspace bytes", 0 if w.workspace is None else w.workspace.numel())
        pu.assert_out_close(pu.out_tensor_bits(out), ref["out_bits"], False,
                            pu.reorder_bound(ref["acc"], scales, ref["s_a"]), f"workspace reuse M={M}")
    assert int(w.workspace[:65536].view(torch.int32).abs().max()) == 0   # the counter block is back at zero


def test_config_c5_asym_ragged(gpu_ops, oracle):
    a, b = workloads.config_cases("c5")
    _run_case(gpu_ops, oracle, a, "auto")                  # M = 77, per-group zero-points: whichever kernel AUTO routes it to
    _run_case(gpu_ops, oracle, b, "auto")                  # M = 1  -> skinny split-K


def test_wint2_gemm_and_linear_entry_points(gpu_ops, oracle):
    case = pu.small_case(5, 128, 256, 128, "sym", seed=9)
    packed, scales, zero = pu.quantized_weight(case)
    x = workloads.make_activation(case)
    ref = oracle.reference_forward(x, packed, scales, zero, 128)
    xd = torch.from_numpy(x).cuda()
    y = gpu_ops.wint2_gemm(xd, torch.from_numpy(packed).cuda().t(), torch.from_numpy(scales).cuda())
    pu.assert_out_close(pu.out_tensor_bits(y), ref["out_bits"], False,
                        pu.reorder_bound(ref["acc"], scales, ref["s_a"]), "wint2_gemm")
    lin = gpu_ops.W2A8Linear.from_float(workloads.make_weight(case).astype(np.float32), 128, "sym")
    y2 = lin(xd.reshape(1, 5, 256))
    assert y2.shape == (1, 5, 128)
    np.testing.assert_array_equal(pu.out_tensor_bits(y2.reshape(5, 128)), pu.out_tensor_bits(y))


def test_wint2_gemm_keeps_the_repacked_weight_until_it_changes(gpu_ops, oracle):
    from slimkernels_amd.torch import ops as ops_mod
    case = pu.small_case(3, 192, 512, 128, "sym", seed=21)
    packed, scales, zero = pu.quantized_weight(case)
    x = workloads.make_activation(case)
    xd = torch.from_numpy(x).cuda()
    wt, sc = torch.from_numpy(packed).cuda().t(), torch.from_numpy(scales).cuda()
    ops_mod._WINT2_CACHE.clear()
    y1 = gpu_ops.wint2_gemm(xd, wt, sc)
    assert len(ops_mod._WINT2_CACHE) == 1
    held = next(iter(ops_mod._WINT2_CACHE.values()))[0]
    y2 = gpu_ops.wint2_gemm(xd, wt, sc)
    assert len(ops_mod._WINT2_CACHE) == 1 and next(iter(ops_mod._WINT2_CACHE.values()))[0] is held
    assert torch.equal(y1, y2)
    # the documented call form makes a new view object per call: wint2_gemm(x, packed.t(), scale) must hit as well
    pk = torch.from_numpy(packed).cuda()
    ops_mod._WINT2_CACHE.clear()
    ya = gpu_ops.wint2_gemm(xd, pk.t(), sc)
    held_t = next(iter(ops_mod._WINT2_CACHE.values()))[0]
    yb = gpu_ops.wint2_gemm(xd, pk.t(), sc)
    assert len(ops_mod._WINT2_CACHE) == 1 and next(iter(ops_mod._WINT2_CACHE.values()))[0] is held_t
    assert torch.equal(ya, yb) and torch.equal(ya, y1)
    # operands made under inference mode have no version counter to read: re-laid every call, same result
    with torch.inference_mode():
        pk_i, sc_i = torch.from_numpy(packed).cuda(), torch.from_numpy(scales).cuda()
        yi = gpu_ops.wint2_gemm(xd, pk_i.t(), sc_i)
    assert torch.equal(yi, y1)
    ref = oracle.reference_forward(x, packed, scales, zero, 128)
    pu.assert_out_close(pu.out_tensor_bits(y2), ref["out_bits"], False, pu.reorder_bound(ref["acc"], scales, ref["s_a"]), "wint2 cached")
    # an in-place change of the packed weight is seen (version counter): re-laid, new result
    packed2 = packed.copy()
    packed2[:, :8] ^= 0x55
    wt.copy_(torch.from_numpy(packed2).cuda().t())
    y3 = gpu_ops.wint2_gemm(xd, wt, sc)
    ref3 = oracle.reference_forward(x, packed2, scales, zero, 128)
    pu.assert_out_close(pu.out_tensor_bits(y3), ref3["out_bits"], False, pu.reorder_bound(ref3["acc"], scales, ref3["s_a"]), "wint2 changed")
    assert not torch.equal(y3, y1)
    for _ in range(40):   # the cache stays small
        gpu_ops.wint2_gemm(xd, wt.clone(), sc)
    assert len(ops_mod._WINT2_CACHE) <= ops_mod._WINT2_CACHE_SIZE


def test_split_k_workspaces_are_per_stream(gpu_ops, oracle):
    """A weight used on two streams gets a workspace for each (calls that share one must not overlap in time)."""
    case = pu.small_case(16, 128, 14336, 128, "sym", seed=4)
    packed, scales, zero = pu.quantized_weight(case)
    x = workloads.make_activation(case)
    w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
    qa = gpu_ops.quantize_act_int8(xd, 128)
    y0 = gpu_ops.w2a8_gemm(qa, w, kernel="skinny", split_k=4)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        y1 = gpu_ops.w2a8_gemm(qa, w, kernel="skinny", split_k=4)
    side.synchronize()
    assert len(w.workspaces) == 2
    a, b = w.workspaces.values()
    assert a.data_ptr() != b.data_ptr()
    assert torch.equal(y0, y1)


def test_grouped_launch_matches_single_launches(gpu_ops, oracle):
    """One grouped launch over problems of different M, N, K against the oracle, and against the same
    problems launched one by one (another kernel body with another fp32 summation order: the two may
    differ by the re-association noise the oracle comparison admits, not more)."""
    shapes = [(1, 256, 512), (5, 100, 1024), (16, 512, 256), (32, 192, 768), (2, 64, 2048)]
    probs, singles, refs = [], [], []
    for i, (M, N, K) in enumerate(shapes):
        case = pu.small_case(M, N, K, 128, "sym", seed=50 + i)
        packed, scales, zero = pu.quantized_weight(case)
        x = workloads.make_activation(case)
        w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
        qa = gpu_ops.quantize_act_int8(xd, 128)
        probs.append((qa, w))
        singles.append(gpu_ops.w2a8_gemm(qa, w, kernel="skinny", split_k=1))
        refs.append((oracle.reference_forward(x, packed, scales, zero, 128), scales))
    outs = gpu_ops.w2a8_gemm_grouped(probs)
    torch.cuda.synchronize()
    for o, s, (ref, scales) in zip(outs, singles, refs):
        bound = pu.reorder_bound(ref["acc"], scales, ref["s_a"])
        pu.assert_out_close(pu.out_tensor_bits(o), ref["out_bits"], False, bound, "grouped")
        pu.assert_out_close(pu.out_tensor_bits(o), pu.out_tensor_bits(s), False, 2 * bound, "grouped vs single")
    # asymmetric group, bf16
    case = pu.small_case(7, 130, 512, 64, "asym", seed=77, out_dtype="bfloat16")
    packed, scales, zero = pu.quantized_weight(case)
    x = workloads.make_activation(case)
    w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
    qa = gpu_ops.quantize_act_int8(xd, 64)
    (o,) = gpu_ops.w2a8_gemm_grouped([(qa, w)], torch.bfloat16)
    ref = oracle.reference_forward(x, packed, scales, zero, 64, out_bf16=True)
    pu.assert_out_close(pu.out_tensor_bits(o), ref["out_bits"], True, pu.reorder_bound(ref["acc"], scales, ref["s_a"]), "grouped asym")


def test_grouped_launch_that_fills_the_chip(gpu_ops, oracle):
    """A launch of more than 512 workgroups keeps the default k-parts (1 / 2 / 4 by K: the shared-
    activation bodies with 8, 4 and 2 strips per workgroup) for the problems of its first round and
    doubles them for the problems that start later; a small launch raises them all.  Three weights,
    each used by problems of several M, every output against the oracle."""
    weights = {}
    for name, (N, K) in {"a": (8192, 4096), "b": (8192, 2048), "c": (4096, 14336)}.items():
        case = pu.small_case(1, N, K, 128, "sym", seed=900 + K)
        packed, scales, zero = pu.quantized_weight(case)
        w, _ = pu.device_inputs(gpu_ops, case, packed, scales, zero, workloads.make_activation(case))
        weights[name] = (N, K, packed, scales, zero, w)
    plan = [("c", 1), ("c", 16), ("c", 32)] + [("a", m) for m in (1, 3, 8, 16, 32, 2, 4, 12, 24)] + \
           [("b", m) for m in (1, 3, 8, 16, 32)]
    probs, refs = [], []
    for i, (name, M) in enumerate(plan):
        N, K, packed, scales, zero, w = weights[name]
        case = pu.small_case(M, N, K, 128, "sym", seed=950 + i)
        x = workloads.make_activation(case)
        xd = torch.from_numpy(x).cuda()
        probs.append((gpu_ops.quantize_act_int8(xd, 128), w))
        refs.append((oracle.reference_forward(x, packed, scales, zero, 128), scales))
    _say("grouped launch of", len(probs), "problems")
    outs = gpu_ops.w2a8_gemm_grouped(probs)
    torch.cuda.synchronize()
    for (name, M), o, (ref, scales) in zip(plan, outs, refs):
        pu.assert_out_close(pu.out_tensor_bits(o), ref["out_bits"], False,
                            pu.reorder_bound(ref["acc"], scales, ref["s_a"]), f"grouped big launch {name} M={M}")


# shape classes of the grouped kernel in small launches (k-parts raised to 4 / 8 where K allows): one-row /
# few-row / shared-activation bodies (by M), two row blocks (M > 16), group sizes 64 / 128 / 256, per-group
# zero-points, a K range whose last chunk is ragged, k-parts of unequal length
GROUPED_SETS = [
    (128, "sym", [(1, 192, 8192), (9, 192, 8192), (32, 130, 14336), (4, 64, 14336), (16, 300, 4096), (17, 64, 4096)]),
    (64, "sym", [(1, 128, 8192), (12, 128, 2368), (32, 100, 6208)]),
    (256, "sym", [(3, 100, 3328), (16, 64, 25600)]),
    (128, "asym", [(20, 64, 13824), (1, 130, 13824), (8, 96, 4096)]),
    (64, "asym", [(16, 64, 2368), (2, 64, 8192)]),
]


@pytest.mark.gpu
@pytest.mark.parametrize("g,mode,shapes", GROUPED_SETS)
def test_grouped_kernel_shape_classes(gpu_ops, oracle, g, mode, shapes):
    probs, refs = [], []
    for i, (M, N, K) in enumerate(shapes):
        case = pu.small_case(M, N, K, g, mode, seed=300 + 7 * i + g)
        packed, scales, zero = pu.quantized_weight(case)
        x = workloads.make_activation(case)
        w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
        probs.append((gpu_ops.quantize_act_int8(xd, g), w))
        refs.append((oracle.reference_forward(x, packed, scales, zero, g), scales))
    outs = gpu_ops.w2a8_gemm_grouped(probs)
    torch.cuda.synchronize()
    for (M, N, K), o, (ref, scales) in zip(shapes, outs, refs):
        pu.assert_out_close(pu.out_tensor_bits(o), ref["out_bits"], False,
                            pu.reorder_bound(ref["acc"], scales, ref["s_a"]), f"grouped {M}x{N}x{K} g{g} {mode}")


# ------------------------------------------------------------------ activation quantisation inside the GEMM
@pytest.mark.parametrize("M,N,K,g,mode,xdt,out,split", [
    (1, 4096, 4096, 128, "sym", "float16", "float16", 0),
    (1, 100, 256, 64, "asym", "bfloat16", "bfloat16", 0),
    (2, 192, 14336, 128, "sym", "float16", "float16", 0),      # long K, few strips: K split across workgroups
    (3, 640, 8192, 256, "asym", "float16", "bfloat16", 2),
    (4, 1024, 8192, 64, "ref", "bfloat16", "float16", 1),
    (4, 64, 2368, 64, "sym", "float16", "float16", 0),         # 37 steps: a ragged last chunk
    (1, 5120, 28672, 64, "sym", "float16", "bfloat16", 0),
    # more than four rows, or rows too long for LDS: the grid's first workgroups quantise them into the workspace
    (5, 4096, 4096, 128, "sym", "float16", "float16", 0),
    (4, 256, 14336, 128, "sym", "float16", "float16", 0),      # few rows, but 56 KiB of them; K split across workgroups
    (16, 1000, 4096, 64, "asym", "bfloat16", "bfloat16", 0),
    (17, 130, 8192, 128, "ref", "float16", "float16", 1),      # two row blocks, activations fetched two steps wide
    (32, 4096, 4096, 128, "sym", "float16", "bfloat16", 0),
    (32, 192, 14336, 128, "asym", "float16", "float16", 0),
    (24, 64, 512, 256, "asym", "float16", "float16", 0),       # a grid of two workgroups for 24 rows: several rows each
    (9, 64, 2368, 64, "sym", "bfloat16", "float16", 0),        # 37 steps: a ragged last chunk
])
def test_fused_activation_quantisation_matches_two_launches(gpu_ops, oracle, M, N, K, g, mode, xdt, out, split):
    """Up to 32 token rows: slimk_w2a8_gemm_fused quantises the rows inside the GEMM launch.  Same
    bits as act-quant followed by the skinny kernel with the same split, and the oracle's output."""
    _say("fused", M, N, K, g, mode, xdt, out, split)
    case = pu.small_case(M, N, K, g, mode, seed=M + N + K, out_dtype=out)
    packed, scales, zero = pu.quantized_weight(case)
    x = workloads.make_activation(case)
    w, xd = pu.device_inputs(gpu_ops, case, packed, scales, zero, x)
    if xdt == "bfloat16":
        xd = xd.to(torch.bfloat16)
        x = xd.float().cpu().numpy().astype(np.float32)
    odt = pu.torch_dtype(case)
    fused = gpu_ops.w2a8_linear_fused(xd, w, odt, split_k=split)
    two = gpu_ops.w2a8_gemm(gpu_ops.quantize_act_int8(xd, g), w, odt, kernel="skinny", split_k=split)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(pu.out_tensor_bits(fused), pu.out_tensor_bits(two))
    # against the oracle as well (bf16 rows go to it as bit patterns)
    x_or_bits = pu.out_tensor_bits(xd) if xdt == "bfloat16" else x
    ref = oracle.reference_forward(x_or_bits, packed, scales, zero, g, out_bf16=(out == "bfloat16"), want_acc=True,
                                   x_bf16=(xdt == "bfloat16"))
    pu.assert_out_close(pu.out_tensor_bits(fused), ref["out_bits"], out == "bfloat16",
                        pu.reorder_bound(ref["acc"], scales, ref["s_a"]), case.name)
    # a strided view of a wider buffer, and the layer's forward (which picks the fused path for few rows)
    wide = torch.zeros(M, K + 16, dtype=xd.dtype, device="cuda")
    wide[:, :K] = xd
    np.testing.assert_array_equal(pu.out_tensor_bits(gpu_ops.w2a8_linear_fused(wide[:, :K], w, odt, split_k=split)),
                                  pu.out_tensor_bits(fused))
    lin = gpu_ops.W2A8Linear(w, None, odt)
    np.testing.assert_array_equal(pu.out_tensor_bits(lin(xd)), pu.out_tensor_bits(
        gpu_ops.w2a8_gemm(gpu_ops.quantize_act_int8(xd, g), w, odt)))
    with pytest.raises(ValueError):
        gpu_ops.w2a8_linear_fused(torch.zeros(33, K, dtype=xd.dtype, device="cuda"), w, odt)
    if M > 4 or M * K > 32768:
        # the bounded wait: with no polls at all every workgroup quantises the rows itself; with few, some do
        from slimkernels_amd import _lib
        for polls in (0, 3):
            old = _lib.lib().slimk_w2a8_set_fused_spin_limit(polls)
            try:
                again = gpu_ops.w2a8_linear_fused(xd, w, odt, split_k=split)
                torch.cuda.synchronize()
            finally:
                _lib.lib().slimk_w2a8_set_fused_spin_limit(old)
            np.testing.assert_array_equal(pu.out_tensor_bits(again), pu.out_tensor_bits(fused))
        # and the workspace is left ready for the next call, of this or another kind
        np.testing.assert_array_equal(pu.out_tensor_bits(gpu_ops.w2a8_linear_fused(xd, w, odt, split_k=split)), pu.out_tensor_bits(fused))
        np.testing.assert_array_equal(pu.out_tensor_bits(gpu_ops.w2a8_gemm(gpu_ops.quantize_act_int8(xd, g), w, odt, kernel="skinny", split_k=split)),
                                      pu.out_tensor_bits(two))
