"""W4A8 through the W2A8 kernels: a 4-bit weight is held as two 2-bit planes over a reduction of 2K
(see slimkernels_amd/w4.py for the identity), the activation row is laid down twice, and every GEMM is one
launch of the W2 kernels.  Upstream's only W4 code is the notebook kernel ``w4matmul_splitk(a, b, c)``
(slimkernels/triton/gemm_splitk.ipynb cell 0); its call form is mirrored at the bottom."""
from __future__ import annotations

import dataclasses
from typing import Optional

import numpy as np
import torch

from .. import w4 as host_w4
from .. import _lib
from .ops import (QuantizedActivation, W2A8Weight, _DT, _require_cuda, _stream_ptr, _workspace, fused_applies, quantize_act_int8, repack_w2,
                  w2a8_gemm, w2a8_linear_fused)


@dataclasses.dataclass
class W4A8Weight:
    """A 4-bit weight [N, K] as the W2 operand over 2K (hi plane, then lo plane)."""
    planes: W2A8Weight
    N: int
    K: int
    group_size: int
    uniform_zp8: bool = False   # every zero-point is 8 (the symmetric levels): the one-pass kernel needs no row sums

    @property
    def device(self):
        return self.planes.device


def repack_w4(packed4, scales, zp=None, group_size: int = 128, zp_const: int = 8, device="cuda") -> W4A8Weight:
    """packed4: uint8 [N, K/2] (pack_w4 layout), scales: float16 [G, N], zp: uint8 [G, N] with values 0..15 or
    None for a uniform zero-point ``zp_const`` (8: the symmetric levels -8..7).  numpy arrays or tensors."""
    packed4 = packed4.cpu().numpy() if isinstance(packed4, torch.Tensor) else np.asarray(packed4)
    scales = scales.cpu().numpy() if isinstance(scales, torch.Tensor) else np.asarray(scales)
    if packed4.dtype != np.uint8 or packed4.ndim != 2:
        raise ValueError("packed4 must be a 2-D uint8 array [N, K/2]")
    N, K = packed4.shape[0], packed4.shape[1] * 2
    if scales.dtype != np.float16 or scales.ndim != 2 or K % group_size != 0 or scales.shape != (K // group_size, N):
        raise ValueError(f"scales must be float16 [K/group_size, N] = {(K // max(group_size, 1), N)}")
    if zp is None:
        if not 0 <= int(zp_const) <= 15:
            raise ValueError("zp_const must be in 0..15")
        zp = np.full(scales.shape, int(zp_const), dtype=np.uint8)
    else:
        zp = zp.cpu().numpy() if isinstance(zp, torch.Tensor) else np.asarray(zp)
    packed2, scales2, zp2 = host_w4.split_planes(host_w4.unpack_w4(packed4), scales, zp)
    return W4A8Weight(repack_w2(packed2, scales2, zp2, group_size, device=device), N, K, group_size,
                      uniform_zp8=bool((zp == 8).all()))


def quantize_weight4_gpu(weight_nk: torch.Tensor, group_size: int = 128, mode: str = "sym"):
    """Group-wise 4-bit quantisation of an fp16 / bf16 weight [N, K] on the GPU, as the two 2-bit planes over 2K:
    the same numbers as ``split_planes(unpack_w4(...prepare_w4(weight)))`` on the host.  Returns (planes uint8
    [N, 2K/4], scales float16 [2G, N], zero-points uint8 [2G, N]) as device tensors, the inputs of repack_w2."""
    L = _lib.lib()
    _require_cuda(weight_nk, "weight")
    if weight_nk.dim() != 2 or weight_nk.dtype not in _DT:
        raise ValueError("weight must be a 2-D float16 or bfloat16 tensor [N, K]")
    modes = {"sym": _lib.QUANT_SYM, "asym": _lib.QUANT_ASYM}
    if mode not in modes:
        raise ValueError(f"unknown quantizer mode {mode!r} (expected 'sym' or 'asym')")
    w = weight_nk if weight_nk.stride(1) == 1 and weight_nk.stride(0) % 8 == 0 and weight_nk.data_ptr() % 16 == 0 \
        else weight_nk.contiguous()
    N, K = w.shape
    if group_size not in (64, 128, 256) or K % group_size != 0:
        raise ValueError(f"unsupported K={K}, group_size={group_size} (group_size in (64, 128, 256), K % group_size == 0)")
    dev = w.device
    G = K // group_size
    planes = torch.empty((N, K // 2), dtype=torch.uint8, device=dev)
    scales2 = torch.empty((2 * G, N), dtype=torch.float16, device=dev)
    zp2 = torch.empty((2 * G, N), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _lib.check(L.slimk_w2a8_quantize_weight4(w.data_ptr(), w.stride(0), _DT[w.dtype], N, K, group_size, modes[mode],
                                                 planes.data_ptr(), planes.stride(0), scales2.data_ptr(), zp2.data_ptr(),
                                                 _stream_ptr(dev)))
        if w is not weight_nk:
            torch.cuda.current_stream(dev).synchronize()  # the contiguous copy is consumed by the enqueued kernel
    return planes, scales2, zp2


def save_w4(path, packed4, scales, zp=None, group_size: int = 128, zp_const: int = 8):
    """Write a 4-bit weight to the on-disk container of slimkernels_amd.packed_format as its two 2-bit planes over
    2K (mode tag "w4planes"): the file holds what the W2 entry points consume, in the interchange layout."""
    from ..packed_format import save_w2
    packed4 = np.asarray(packed4)
    scales = np.asarray(scales)
    if zp is None:
        zp = np.full(scales.shape, int(zp_const), dtype=np.uint8)
    packed2, scales2, zp2 = host_w4.split_planes(host_w4.unpack_w4(packed4), scales, np.asarray(zp))
    save_w2(path, packed2, scales2, zp2, group_size, mode="w4planes")


def load_w4_weight(path, device="cuda", mmap=True) -> W4A8Weight:
    """A file written by save_w4 -> the weight on the GPU."""
    from ..packed_format import load_w2
    d = load_w2(path, mmap=mmap)
    if d["mode"] != "w4planes" or d["zp"] is None or d["K"] % 2 != 0:
        raise ValueError(f"{path}: not a two-plane W4 file (mode {d['mode']!r})")
    planes = repack_w2(d["packed"], d["scales"], d["zp"], d["group_size"], device=device)
    G = d["K"] // 2 // d["group_size"]
    zp = np.asarray(d["zp"])
    return W4A8Weight(planes, d["N"], d["K"] // 2, d["group_size"],
                      uniform_zp8=bool((zp[:G] == 2).all() and (zp[G:] == 0).all()))


def activation_twice(qa: QuantizedActivation) -> QuantizedActivation:
    """The activation operand over 2K: the int8 row and its per-group sums laid down twice."""
    return QuantizedActivation(torch.cat([qa.q, qa.q], dim=1), qa.s_a, torch.cat([qa.rowsum, qa.rowsum], dim=0),
                               qa.group_size)


def w4a8_gemm(qa: QuantizedActivation, w: W4A8Weight, out_dtype=torch.float16, *, kernel: str = "auto",
              split_k: int = 0, dump: Optional[str] = None, out: Optional[torch.Tensor] = None):
    """out[M, N] = dequant( q @ (codes4 - zp4)^T ) for ``qa`` = quantize_act_int8(x) over K.  With ``dump`` =
    "groups" also returns the int32 accumulators [M, N, G] (4 * hi-plane + lo-plane sums, exact)."""
    M, K = qa.q.shape
    if K != w.K or qa.group_size != w.group_size:
        raise ValueError(f"activation K={K}/group {qa.group_size} does not match weight K={w.K}/group {w.group_size}")
    if dump not in (None, "groups"):
        raise ValueError("dump must be None or 'groups'")
    res = w2a8_gemm(activation_twice(qa), w.planes, out_dtype, kernel=kernel, split_k=split_k, dump=dump, out=out)
    if dump is None:
        return res
    y, acc = res
    G = K // w.group_size
    return y, acc[:, :, :G] * 4 + acc[:, :, G:]


# Up to 32 token rows the few-rows kernels over the two planes are faster; beyond, the one-pass kernel is (measured
# at M = 33 / 64 / 256: 14336 x 4096 18.5 / 19.1 / 34.6 us against 26.8 / 27.6 / 55.4 us over two planes,
# 4096 x 14336 25.3 / 25.9 / 36.1 us against 36.0 / 36.1 / 53.5 us; at M = 24 it loses, 18.5 us against 15.6 us).
ONE_PASS_MIN_ROWS = 33


def one_pass_applies(M: int, w: W4A8Weight) -> bool:
    return M >= ONE_PASS_MIN_ROWS and w.K % 128 == 0 and w.group_size in (64, 128)


def w4a8_gemm_one_pass(qa: QuantizedActivation, w: W4A8Weight, out_dtype=torch.float16,
                       out: Optional[torch.Tensor] = None, split_k: int = 0) -> torch.Tensor:
    """The many-rows kernel for 4-bit weights: hi and lo digit are put together in front of the
    matrix core, one pass over K (split over several workgroups per tile when the tiles are few; 0 = choose).
    ``qa`` = quantize_act_int8(x) over K (laid down once)."""
    M, K = qa.q.shape
    if K != w.K or qa.group_size != w.group_size:
        raise ValueError(f"activation K={K}/group {qa.group_size} does not match weight K={w.K}/group {w.group_size}")
    if out_dtype not in _DT:
        raise ValueError("out_dtype must be torch.float16 or torch.bfloat16")
    dev = qa.q.device
    if out is None:
        out = torch.empty((M, w.N), dtype=out_dtype, device=dev)
    L = _lib.lib()
    with torch.cuda.device(dev):
        ws = _workspace(w.planes, L.slimk_w4a8_gemm_workspace_bytes(M, w.N, K, w.group_size, split_k))
        # zero-points other than 8 enter through the row sums of the activations
        zp_r = None if w.uniform_zp8 else w.planes.zp_r
        _lib.check(L.slimk_w4a8_gemm(qa.q.data_ptr(), qa.q.stride(0), qa.s_a.data_ptr(),
                                     qa.rowsum.data_ptr() if zp_r is not None else None, qa.rowsum.stride(0),
                                     w.planes.w_r.data_ptr(), w.planes.s_r.data_ptr(),
                                     zp_r.data_ptr() if zp_r is not None else None, M, w.N, K, w.group_size, out.data_ptr(),
                                     out.stride(0), _DT[out.dtype], ws.data_ptr() if ws is not None else None,
                                     ws.numel() if ws is not None else 0, split_k, _stream_ptr(dev)))
    return out


def w4a8_gemm_grouped(problems, out_dtype=torch.float16):
    """Several independent W4A8 GEMMs of at most 32 token rows in ONE launch (the grouped kernel of the W2 path):
    ``problems`` is a list of (qa, w4, out) with ``qa`` = quantize_act_int8(x) over K, ``w4`` a W4A8Weight and
    ``out`` [M, N] of ``out_dtype``.  All problems share the group size."""
    from .ops import w2a8_gemm_grouped
    return w2a8_gemm_grouped([(activation_twice(qa), w.planes, out) for qa, w, out in problems], out_dtype)


def w4a8_linear(x: torch.Tensor, w: W4A8Weight, out_dtype=torch.float16) -> torch.Tensor:
    """x [M, K] fp16 / bf16 -> out [M, N]; one token row goes through the single-launch kernel that quantises
    the row itself."""
    _require_cuda(x, "x")
    if x.dim() != 2 or x.dtype not in _DT:
        raise ValueError("x must be a 2-D float16 or bfloat16 tensor [M, K]")
    if x.shape[1] != w.K:
        raise ValueError(f"activation K={x.shape[1]} does not match weight K={w.K}")
    if x.shape[0] == 1 and fused_applies(1, 2 * w.K):
        return w2a8_linear_fused(torch.cat([x, x], dim=1), w.planes, out_dtype)
    if one_pass_applies(x.shape[0], w):
        return w4a8_gemm_one_pass(quantize_act_int8(x, w.group_size), w, out_dtype)
    # one quantisation launch writes the row and its group sums twice: the operand over 2K
    return w2a8_gemm(quantize_act_int8(x, w.group_size, copies=2), w.planes, out_dtype)


class W4A8Linear(torch.nn.Module):
    """y = x @ W^T with W held as 4-bit codes (+ optional bias), a swap-in for nn.Linear."""

    def __init__(self, weight: W4A8Weight, bias: Optional[torch.Tensor] = None, out_dtype=torch.float16):
        super().__init__()
        self.weight = weight
        self.bias = bias
        self.out_dtype = out_dtype
        self.in_features, self.out_features = weight.K, weight.N

    @classmethod
    def from_float(cls, weight_nk, group_size=128, mode="sym", bias=None, out_dtype=torch.float16, device="cuda"):
        if isinstance(weight_nk, torch.Tensor) and weight_nk.is_cuda and weight_nk.dtype in _DT:
            # quantise where the weight already is (same numbers as the host path)
            planes, scales2, zp2 = quantize_weight4_gpu(weight_nk.detach(), group_size, mode)
            if not bool(torch.isfinite(scales2).all()):
                raise ValueError("4 * scale overflows float16")
            N, K = weight_nk.shape
            return cls(W4A8Weight(repack_w2(planes, scales2, zp2, group_size, device=weight_nk.device), N, K, group_size,
                                  uniform_zp8=mode == "sym"), bias, out_dtype)
        w_np = weight_nk.detach().float().cpu().numpy() if isinstance(weight_nk, torch.Tensor) else np.asarray(weight_nk)
        packed4, scales, zero = host_w4.prepare_w4(w_np, group_size, mode)
        return cls(repack_w4(packed4, scales, zero, group_size, device=device), bias, out_dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        if x2.dtype not in _DT:
            x2 = x2.to(self.out_dtype)
        y = w4a8_linear(x2, self.weight, self.out_dtype)
        if self.bias is not None:
            y = y + self.bias
        return y.reshape(*lead, self.out_features)


def w4matmul_splitk(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor) -> torch.Tensor:
    """The call form of the upstream notebook kernel (gemm_splitk.ipynb cell 0): ``a`` [M, K] fp16, ``b`` the
    packed weight [K/8, N] (eight 4-bit codes per 32-bit word along K, code k % 8 at bits 4 * (k % 8)),
    ``c`` [M, N] fp16, which receives ``c += a @ codes`` -- the raw codes 0..15 are the weight values, there
    are no scales and no zero-point.  Here the product runs as W4A8 (``a`` is quantised per token row to int8),
    so it agrees with the fp16 product to the activation quantisation error.  Repacks on every call."""
    _require_cuda(a, "a")
    codes = host_w4.codes_from_uint32_kn(b.cpu().numpy() if isinstance(b, torch.Tensor) else b)   # [N, K]
    N, K = codes.shape
    if a.shape[1] != K or tuple(c.shape) != (a.shape[0], N):
        raise ValueError(f"shapes do not agree: a {tuple(a.shape)}, b unpacks to K={K}, N={N}, c {tuple(c.shape)}")
    group = 128 if K % 128 == 0 else 64
    ones = np.ones((K // group, N), dtype=np.float16)
    w = repack_w4(host_w4.pack_w4(codes), ones, None, group, zp_const=0, device=a.device)
    c += w4a8_linear(a if a.dtype in _DT else a.half(), w, c.dtype if c.dtype in _DT else torch.float16).to(c.dtype)
    return c
