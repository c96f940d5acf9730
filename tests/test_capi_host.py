"""Host-side checks of the C ABI (no GPU): the library loads, exports every symbol the header
declares, answers its size queries, and rejects bad arguments with the documented codes before
anything could be launched."""
import ctypes
import os
import re
import threading

import pytest

from slimkernels_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "slimk_w2a8.h")
FAKE = 0x10000  # a non-NULL, 16-byte aligned value: validation never dereferences pointers


@pytest.fixture(scope="module")
def L():
    return _lib.lib()


def declared_symbols():
    text = open(HEADER, encoding="utf-8").read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(slimk_w(?:2a8|2a16|4a8)_\w+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(L):
    names = declared_symbols()
    assert len(names) >= 12
    for n in names:
        assert hasattr(L, n), f"{n} is declared in the header but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert set(_lib.SIGNATURES) == set(names)


def test_version_arch_and_sizes(L):
    assert L.slimk_w2a8_version() == 100
    assert L.slimk_w2a8_arch() == b"gfx950"
    assert L.slimk_w2a8_repacked_weight_bytes(4096, 4096) == 4096 * 4096 // 4
    assert L.slimk_w2a8_repacked_weight_bytes(100, 128) == 2 * 4 * 1024     # two strips (N padded to 128) x one run of four steps (two of them padding)
    assert L.slimk_w2a8_repacked_weight_bytes(64, 576) == 12 * 1024         # nine steps: three runs
    assert L.slimk_w2a8_repacked_scale_bytes(4096, 4096, 128) == 2 * 4096 * 32
    assert L.slimk_w2a8_repacked_zp_bytes(4096, 4096, 128) == 4096 * 32
    assert L.slimk_w2a8_repacked_weight_bytes(4096, 100) == 0               # K % 64
    assert L.slimk_w2a8_repacked_scale_bytes(4096, 4096, 96) == 0           # group size
    assert L.slimk_w2a8_repacked_scale_bytes(4096, 4096 + 64, 128) == 0     # K % group


def test_split_heuristic_and_workspace(L):
    # unsplit: many strips, or a matrix of a few MiB
    assert L.slimk_w2a8_gemm_auto_split_k(16, 14336, 4096, 128, _lib.KERNEL_AUTO) == 1
    assert L.slimk_w2a8_gemm_auto_split_k(1, 4096, 4096, 128, _lib.KERNEL_AUTO) == 1
    assert L.slimk_w2a8_gemm_workspace_bytes(16, 14336, 4096, 128, _lib.KERNEL_AUTO, 0) == 0
    # few strips, long K: split to about 256 workgroups
    s = L.slimk_w2a8_gemm_auto_split_k(16, 4096, 14336, 128, _lib.KERNEL_AUTO)
    assert s == 4
    ws = L.slimk_w2a8_gemm_workspace_bytes(16, 4096, 14336, 128, _lib.KERNEL_AUTO, 0)
    assert ws == 65536 + s * 64 * (16 * 64) * 4     # fixed counter block + split x strips x (16 x 64 fp32 tile)
    # 17..32 tokens run as two blocks of 16 rows: one counter and one tile per (strip, block)
    assert L.slimk_w2a8_gemm_workspace_bytes(32, 4096, 14336, 128, _lib.KERNEL_AUTO, 4) == 65536 + 4 * 64 * 2 * (16 * 64) * 4
    # the tiled kernel splits K only when its 64-row tiles would leave CUs idle
    assert L.slimk_w2a8_gemm_auto_split_k(4096, 14336, 4096, 128, _lib.KERNEL_AUTO) == 1
    s = L.slimk_w2a8_gemm_auto_split_k(512, 4096, 14336, 128, _lib.KERNEL_AUTO)      # 16 x 8 tiles, 112 stages
    assert s == 4
    assert L.slimk_w2a8_gemm_workspace_bytes(512, 4096, 14336, 128, _lib.KERNEL_AUTO, 0) == 65536 + s * 128 * (64 * 256) * 4
    assert L.slimk_w2a8_gemm_auto_split_k(0, 4096, 4096, 128, 0) == 0


def test_auto_route(L):
    """Which kernel form AUTO takes: 1 one-strip skinny, 2 tiled, 3 shared-activation skinny, 4 the 33..128-row kernel."""
    route = L.slimk_w2a8_gemm_auto_route
    assert route(1, 4096, 4096, 128) == 1 and route(11, 28672, 8192, 64) == 1 and route(16, 14336, 8192, 64) == 1
    assert route(12, 28672, 8192, 64) == 3 and route(16, 28672, 8192, 64) == 3   # 12..16 rows on 384 strips and more
    assert route(20, 4096, 4096, 128) == 1          # 17..32 rows: shared only on matrices of 24 MiB or more
    assert route(20, 8192, 14336, 128) == 3
    assert route(33, 4096, 4096, 128) == 1          # few workgroups: the one-strip kernel
    assert route(77, 11008, 4096, 128) == 3         # five row blocks on 172 strips: the shared-activation workgroups
    assert route(64, 4096, 14336, 128) == 3         # long reduction, few 256-channel tiles
    assert route(128, 28672, 8192, 64) == 2
    # 33..256 rows: the smallest of four predicted times.  Rows that leave 64-row tiles partly empty on a large matrix:
    # every row of a row part in one workgroup; tiles that fill: the tiled kernel
    assert route(33, 28672, 8192, 64) == 4 and route(48, 8192, 28672, 128) == 4 and route(80, 16384, 16384, 128) == 4
    assert route(49, 28672, 8192, 64) == 2 and route(64, 28672, 8192, 64) == 2 and route(97, 28672, 8192, 64) == 2
    assert route(88, 28672, 8192, 64) == 4 and route(144, 28672, 8192, 128) == 4 and route(161, 28672, 8192, 128) == 2
    assert route(40, 7168, 16384, 64) == 3 and route(72, 20480, 8192, 64) == 3       # a set of strips per CU or fewer, long reduction
    assert route(40, 14336, 4096, 128) in (1, 3) and route(40, 10240, 8192, 128) in (1, 3)   # smaller matrices stay skinny
    assert route(257, 4096, 4096, 128) == 2 and route(2048, 4096, 4096, 128) == 2
    # an explicit request for the skinny kernel on a shape AUTO gives to the tiled one takes the faster skinny form:
    # here the shared-activation workgroups (unsplit; the one-strip form would split K three ways)
    assert route(256, 5120, 13824, 128) == 2 and L.slimk_w2a8_gemm_auto_split_k(256, 5120, 13824, 128, _lib.KERNEL_SKINNY) == 1
    assert route(100, 14336, 2048, 128) in (1, 2)   # reductions of up to 2048 never take the shared form
    assert route(0, 4096, 4096, 128) == 0 and route(16, 4096, 4000, 128) == 0 and route(16, 4096, 4096, 96) == 0


def test_auto_route_only_names_kernels_that_take_the_shape(L):
    """Whatever kernel the fitted choice names for a random shape of 1..300 rows, that kernel accepts the shape: an
    explicit request for it with two K splits and a workspace of 16 bytes passes validation: it stops at the workspace
    check (error 5) or, where two splits come to one, at the launch (error 6 on a machine without a GPU, which is why
    the test only runs there: the pointers are fake).  The workspace size the library quotes for its own choice agrees
    with its split."""
    import random
    import torch
    if torch.cuda.device_count() > 0:
        pytest.skip("fake pointers: only where a launch cannot happen")
    rng = random.Random(20)
    explicit = {1: _lib.KERNEL_SKINNY, 3: _lib.KERNEL_SKINNY, 2: _lib.KERNEL_TILED, 4: _lib.KERNEL_MID}
    seen = set()
    for _ in range(3000):
        g = rng.choice([64, 128, 256])
        K = g * rng.randint(4, 28672 // g)
        N = rng.choice([rng.randint(1, 4096), rng.randint(4096, 65536)])
        M = rng.choice([rng.randint(1, 300), rng.choice([16, 17, 32, 33, 96, 97, 256, 257])])
        if M * K > (1 << 31) - 1 or N * (K // 4) > (1 << 31) - 1:
            continue
        r = L.slimk_w2a8_gemm_auto_route(M, N, K, g)
        assert r in (1, 2, 3, 4), (M, N, K, g, r)
        if M <= 32:
            assert r in (1, 3)
        if M > 256:
            assert r == 2
        seen.add(r)
        ldq = (K + 15) // 16 * 16
        rc = _gemm(L, M=M, N=N, K=K, g=g, ldq=ldq, ldo=N, ldr=(M + 3) // 4 * 4, kernel=explicit[r], split=2, ws=FAKE, wsb=16)
        assert rc in (5, 6), (M, N, K, g, r, rc, L.slimk_w2a8_last_error())
        if rc == 6:   # the launch itself, not a launcher that refuses the shape
            assert b"no ROCm-capable device" in L.slimk_w2a8_last_error(), (M, N, K, g, r, L.slimk_w2a8_last_error())
        split = L.slimk_w2a8_gemm_auto_split_k(M, N, K, g, _lib.KERNEL_AUTO)
        assert split >= 1
        assert (L.slimk_w2a8_gemm_workspace_bytes(M, N, K, g, _lib.KERNEL_AUTO, 0) > 0) == (split > 1), (M, N, K, g, r, split)
    assert seen == {1, 2, 3, 4}


def _gemm(L, **kw):
    a = dict(q=FAKE, ldq=4096, s_a=FAKE, rowsum=FAKE, ldr=16, w_r=FAKE, s_r=FAKE, zp_r=None, zp_const=2,
             M=16, N=4096, K=4096, g=128, out=FAKE, ldo=4096, odt=0, acc=None, dump=0, ws=None, wsb=0,
             kernel=0, split=0, stream=None)
    a.update(kw)
    return L.slimk_w2a8_gemm(a["q"], a["ldq"], a["s_a"], a["rowsum"], a["ldr"], a["w_r"], a["s_r"], a["zp_r"],
                             a["zp_const"], a["M"], a["N"], a["K"], a["g"], a["out"], a["ldo"], a["odt"], a["acc"],
                             a["dump"], a["ws"], a["wsb"], a["kernel"], a["split"], a["stream"])


def test_gemm_argument_validation(L):
    assert _gemm(L, q=None) == 1 and b"NULL" in L.slimk_w2a8_last_error()
    assert _gemm(L, out=None) == 1
    assert _gemm(L, M=0) == 2
    assert _gemm(L, K=4000) == 2 and b"multiple of 64" in L.slimk_w2a8_last_error()
    assert _gemm(L, g=96) == 2
    assert _gemm(L, K=4096 + 64) == 2
    assert _gemm(L, ldq=100) == 2
    assert _gemm(L, ldo=8) == 2
    assert _gemm(L, ldr=8) == 2
    assert _gemm(L, zp_const=7) == 2
    assert _gemm(L, q=FAKE + 4) == 3
    assert _gemm(L, ldq=4096 + 8) == 3
    assert _gemm(L, ldr=18) == 3
    assert _gemm(L, odt=5) == 4
    assert _gemm(L, kernel=9) == 4
    assert _gemm(L, dump=3) == 4
    assert _gemm(L, dump=1, acc=None) == 1
    assert _gemm(L, M=300, ldr=300, kernel=_lib.KERNEL_SKINNY) == 7                        # the skinny kernel stops at 256 rows
    assert _gemm(L, M=64, ldr=64, kernel=_lib.KERNEL_TILED, split=2) == 5       # valid, but needs a workspace
    assert _gemm(L, M=64, ldr=64, kernel=_lib.KERNEL_TILED, split=2, dump=2, acc=FAKE) == 5   # the verification instantiation splits alike
    # row sums fold zero-points: the tiled kernel with the uniform zero-point 2 reads none, everything else needs them
    assert _gemm(L, rowsum=None) == 1 and b"rowsum" in L.slimk_w2a8_last_error()
    assert _gemm(L, M=64, rowsum=None, kernel=_lib.KERNEL_TILED, zp_const=1) == 1
    assert _gemm(L, M=64, rowsum=None, kernel=_lib.KERNEL_TILED, g=256, split=2) == 5         # any group size: accepted up to the workspace check
    assert _gemm(L, M=64, rowsum=None, kernel=_lib.KERNEL_TILED, split=2) == 5                # accepted up to the workspace check
    # split-K without / with too small a workspace (N = 4096, K = 14336 wants split 4)
    assert _gemm(L, K=14336, ldq=14336) == 5 and b"workspace" in L.slimk_w2a8_last_error()
    assert _gemm(L, K=14336, ldq=14336, ws=FAKE, wsb=1024) == 5
    assert _gemm(L, split=64) == 2                                     # more splits than groups
    # 32-bit buffer offsets: more than 2 GiB of repacked weights is refused, not mis-addressed
    assert _gemm(L, N=1 << 19, ldo=1 << 19, K=1 << 16, ldq=1 << 16) == 7 and b"2 GiB" in L.slimk_w2a8_last_error()


def test_gemm_static_refuses_an_oversized_split_on_the_host(L):
    """The entry point that allocates nothing owns 16 MiB + 64 KiB of workspace: an explicit split beyond it is
    refused before any GPU call (so this runs without a GPU)."""
    assert L.slimk_w2a8_static_workspace_bytes() == (16 << 20) + (64 << 10)
    rc = L.slimk_w2a8_gemm_static(FAKE, 14336, FAKE, FAKE, 512, FAKE, FAKE, None, 2, 512, 4096, 14336, 128,
                                  FAKE, 4096, 0, _lib.KERNEL_TILED, 8, None)
    assert rc == 5 and b"library-owned" in L.slimk_w2a8_last_error()


def test_repack_and_act_quant_validation(L):
    r = L.slimk_w2a8_repack
    assert r(None, 1024, FAKE, None, 4096, 4096, 128, FAKE, FAKE, None, None) == 1
    assert r(FAKE, 1024, FAKE, FAKE, 4096, 4096, 128, FAKE, FAKE, None, None) == 1     # zp without zp_r
    assert r(FAKE, 100, FAKE, None, 4096, 4096, 128, FAKE, FAKE, None, None) == 2      # ldw < K/4
    assert r(FAKE, 1024, FAKE, None, 4096, 4096, 100, FAKE, FAKE, None, None) == 2
    assert r(FAKE, 1024, FAKE, None, 4096, 4096, 128, FAKE + 8, FAKE, None, None) == 3
    a = L.slimk_w2a8_act_quant
    assert a(None, 4096, 0, 1, 4096, 128, FAKE, 4096, FAKE, FAKE, 4, None) == 1
    assert a(FAKE, 4096, 0, 0, 4096, 128, FAKE, 4096, FAKE, FAKE, 4, None) == 2
    assert a(FAKE, 4096, 3, 1, 4096, 128, FAKE, 4096, FAKE, FAKE, 4, None) == 4
    assert a(FAKE, 100, 0, 1, 4096, 128, FAKE, 4096, FAKE, FAKE, 4, None) == 2
    assert a(FAKE, 4096 + 4, 0, 1, 4096, 128, FAKE, 4096, FAKE, FAKE, 4, None) == 3
    assert a(FAKE, 4096, 0, 5, 4096, 128, FAKE, 4096, FAKE, FAKE, 4, None) == 2        # ldr < M
    rep = L.slimk_w2a8_act_quant_rep  # (x, ldx, dtype, M, K, group, copies, q, ldq, s_a, rowsum, ldr, stream)
    assert rep(FAKE, 4096, 0, 1, 4096, 128, 0, FAKE, 8192, FAKE, FAKE, 4, None) == 2
    assert rep(FAKE, 4096, 0, 1, 4096, 128, 5, FAKE, 32768, FAKE, FAKE, 4, None) == 2
    assert rep(FAKE, 4096, 0, 1, 4096, 128, 2, FAKE, 4096, FAKE, FAKE, 4, None) == 2   # ldq < copies * K
    assert b"copies * K" in L.slimk_w2a8_last_error()
    assert rep(None, 4096, 0, 1, 4096, 128, 2, FAKE, 8192, FAKE, FAKE, 4, None) == 1
    qw = L.slimk_w2a8_quantize_weight  # (w, ldw, dtype, N, K, group, mode, packed, ldp, scales, zp, stream)
    assert qw(None, 4096, 0, 64, 4096, 128, 1, FAKE, 1024, FAKE, None, None) == 1
    assert qw(FAKE, 4096, 0, 64, 4096, 128, 2, FAKE, 1024, FAKE, None, None) == 1      # per-group zero-points need zp
    assert qw(FAKE, 4096, 0, 0, 4096, 128, 1, FAKE, 1024, FAKE, None, None) == 2
    assert qw(FAKE, 4096, 0, 64, 4096, 100, 1, FAKE, 1024, FAKE, None, None) == 2
    assert qw(FAKE, 4096, 0, 64, 4096, 128, 1, FAKE, 1000, FAKE, None, None) == 2      # ldp < K/4
    assert qw(FAKE, 4096, 2, 64, 4096, 128, 1, FAKE, 1024, FAKE, None, None) == 4      # dtype
    assert qw(FAKE, 4096, 0, 64, 4096, 128, 3, FAKE, 1024, FAKE, None, None) == 4      # mode
    assert qw(FAKE, 4100, 0, 64, 4096, 128, 1, FAKE, 1024, FAKE, None, None) == 3      # ldw % 8
    assert qw(FAKE, 4096, 0, 64, 4096, 128, 1, FAKE + 1, 1024, FAKE, None, None) == 3
    # (q, ldq, s_a, rowsum, ldr, w_r, s_r, zp_r, M, N, K, group, out, ldo, out_dtype, ws, ws_bytes, split, stream)
    g4 = L.slimk_w4a8_gemm
    assert g4(None, 4096, FAKE, None, 0, FAKE, FAKE, None, 64, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 1, None) == 1
    assert g4(FAKE, 4096, FAKE, None, 64, FAKE, FAKE, FAKE, 64, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 1, None) == 1   # zp_r without row sums
    assert g4(FAKE, 4096, FAKE, FAKE, 60, FAKE, FAKE, FAKE, 64, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 1, None) == 2   # ldr < M
    assert g4(FAKE, 4096, FAKE, FAKE, 66, FAKE, FAKE, FAKE, 64, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 1, None) == 3   # ldr % 4
    assert g4(FAKE, 4096, FAKE, None, 0, FAKE, FAKE, None, 64, 4096, 4096, 256, FAKE, 4096, 0, None, 0, 1, None) == 7    # group 256
    assert g4(FAKE, 4160, FAKE, None, 0, FAKE, FAKE, None, 64, 4096, 4160, 64, FAKE, 4096, 0, None, 0, 1, None) == 7     # K % 128
    assert g4(FAKE, 4000, FAKE, None, 0, FAKE, FAKE, None, 64, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 1, None) == 2    # ldq < K
    assert g4(FAKE, 4096, FAKE, None, 0, FAKE, FAKE, None, 64, 4096, 4096, 128, FAKE, 4096, 3, None, 0, 1, None) == 4
    assert g4(FAKE, 4100, FAKE, None, 0, FAKE, FAKE, None, 64, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 1, None) == 3
    assert g4(FAKE, 4096, FAKE, None, 0, FAKE, FAKE, None, 64, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 4, None) == 5    # split without workspace
    assert g4(FAKE, 4096, FAKE, None, 0, FAKE, FAKE, None, 64, 4096, 4096, 128, FAKE, 4096, 0, FAKE, 1024, 4, None) == 5
    assert g4(FAKE, 4096, FAKE, None, 0, FAKE, FAKE, None, 64, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 33, None) == 2   # more splits than stages
    s4 = L.slimk_w4a8_gemm_auto_split_k(64, 4096, 4096, 128)           # 16 tiles, 32 stages: 4 splits of 8 stages
    assert s4 == 4
    assert L.slimk_w4a8_gemm_workspace_bytes(64, 4096, 4096, 128, 0) == 65536 + 4 * 16 * 64 * 256 * 4
    assert L.slimk_w4a8_gemm_auto_split_k(2048, 14336, 4096, 128) == 1 and L.slimk_w4a8_gemm_workspace_bytes(2048, 14336, 4096, 128, 0) == 0
    assert L.slimk_w4a8_gemm_auto_split_k(64, 4096, 4096, 256) == 0
    q4 = L.slimk_w2a8_quantize_weight4  # (w, ldw, dtype, N, K, group, mode, planes, ldp, scales2, zp2, stream)
    assert q4(FAKE, 4096, 0, 64, 4096, 128, 1, FAKE, 2048, FAKE, None, None) == 1       # zero-points are always written
    assert q4(FAKE, 4096, 0, 64, 4096, 128, 0, FAKE, 2048, FAKE, FAKE, None) == 4       # no REF mode at four bits
    assert q4(FAKE, 4096, 0, 64, 4096, 128, 1, FAKE, 1024, FAKE, FAKE, None) == 2       # ldp < K/2
    assert q4(FAKE, 4096, 0, 0, 4096, 128, 1, FAKE, 2048, FAKE, FAKE, None) == 2
    assert q4(FAKE, 4100, 0, 64, 4096, 128, 2, FAKE, 2048, FAKE, FAKE, None) == 3
    # (x, ldx, dtype, w_r, s_r, zp_r, zp_const, M, N, K, group, out, ldo, out_dtype, ws, ws_bytes, split, stream)
    gf = L.slimk_w2a8_gemm_fused
    assert gf(None, 4096, 0, FAKE, FAKE, None, 2, 1, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 0, None) == 1
    # more than four rows, or rows x K > 32768: the rows go through the workspace, which must be there and big enough
    assert gf(FAKE, 4096, 0, FAKE, FAKE, None, 2, 5, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 0, None) == 5
    assert gf(FAKE, 16384, 0, FAKE, FAKE, None, 2, 4, 4096, 16384, 128, FAKE, 4096, 0, FAKE, 65536, 0, None) == 5
    assert gf(FAKE, 4096, 0, FAKE, FAKE, None, 2, 33, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 0, None) == 7  # more than 32 rows
    fw = L.slimk_w2a8_gemm_fused_workspace_bytes   # (M, N, K, group, split)
    assert fw(1, 4096, 4096, 128, 0) == 0 and fw(4, 4096, 4096, 128, 1) == 0       # in-workgroup form, K unsplit
    assert fw(1, 4096, 14336, 128, 0) == L.slimk_w2a8_gemm_workspace_bytes(1, 4096, 14336, 128, 1, 0)
    assert fw(5, 4096, 4096, 128, 1) == 65536 + 32 * 4096 + 256 + 32 * 32 * 4       # counters, int8 rows, scales, group sums
    assert fw(32, 4096, 4096, 128, 2) == fw(5, 4096, 4096, 128, 1) + 2 * 64 * 2 * 16 * 64 * 4
    assert fw(33, 4096, 4096, 128, 0) == 0 and fw(5, 4096, 4000, 128, 0) == 0
    old = L.slimk_w2a8_set_fused_spin_limit(7)
    assert L.slimk_w2a8_set_fused_spin_limit(old) == 7 and old > 0
    assert gf(FAKE, 4000, 0, FAKE, FAKE, None, 2, 1, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 0, None) == 2   # ldx < K
    assert gf(FAKE, 4100, 0, FAKE, FAKE, None, 2, 1, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 0, None) == 3   # ldx % 8
    assert gf(FAKE, 4096, 2, FAKE, FAKE, None, 2, 1, 4096, 4096, 128, FAKE, 4096, 0, None, 0, 0, None) == 4
    assert gf(FAKE, 14336, 0, FAKE, FAKE, None, 2, 1, 4096, 14336, 128, FAKE, 4096, 0, None, 0, 0, None) == 5  # wants split 4: no workspace
    assert L.slimk_w2a8_workspace_init(None, 64, None) == 1
    assert L.slimk_w2a8_workspace_init(FAKE, 0, None) == 0                             # nothing to do
    assert L.slimk_w2a8_read_probe(FAKE, 24, FAKE, None) == 3


def test_last_error_is_thread_local(L):
    assert _gemm(L, g=96) == 2
    mine = L.slimk_w2a8_last_error()
    seen = {}

    def other():
        seen["before"] = L.slimk_w2a8_last_error()
        _gemm(L, q=None)
        seen["after"] = L.slimk_w2a8_last_error()

    t = threading.Thread(target=other)
    t.start()
    t.join()
    assert seen["before"] == b"" and b"NULL" in seen["after"]
    assert L.slimk_w2a8_last_error() == mine


def test_python_entry_refuses_cpu_tensors():
    import torch
    from slimkernels_amd import torch as ops
    with pytest.raises(ValueError, match="no CPU path"):
        ops.quantize_act_int8(torch.zeros(2, 64, dtype=torch.float16))
    with pytest.raises(ValueError):
        ops.wint2_gemm(torch.zeros(2, 64, dtype=torch.float16), torch.zeros(16, 8, dtype=torch.uint8),
                       torch.zeros(1, 8, dtype=torch.float16))
