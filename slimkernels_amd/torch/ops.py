"""Tensor-level wrappers around the C ABI.

Call pattern of the path (upstream has only the raw launcher
gemm_tn(m, n, a_k, b_k, alpha, A, ldA, B, ldB, beta, C, ldC, stream),
slimkernels/cute/gemm/wgmma_sm90_W2A8.cu:428-437, and the notebook entry
wint2_gemm(activation, weight, scale), triton.ipynb cell 1):

    w  = repack_w2(packed, scales, zp=None, group_size=128)   # once per weight
    qa = quantize_act_int8(x, group_size=128)                 # per forward
    y  = w2a8_gemm(qa, w, out_dtype=torch.float16)            # per forward
    y  = wint2_gemm(x, packed.T, scales)                      # one-shot convenience form

Every function raises if the HIP library is missing or a call fails; nothing here
computes on the CPU.
"""
from __future__ import annotations

import ctypes
import collections
import dataclasses
from typing import Optional

import numpy as np
import torch

from .. import _lib

_DT = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _require_cuda(t: torch.Tensor, name: str):
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got device {t.device}); there is no CPU path")


@dataclasses.dataclass
class W2A8Weight:
    """Weights of one linear layer in the gfx950 streaming layout."""
    w_r: torch.Tensor                 # int32, repacked 2-bit codes
    s_r: torch.Tensor                 # float16, repacked group scales
    zp_r: Optional[torch.Tensor]      # uint8 repacked zero-points, or None (uniform)
    zp_const: int
    N: int
    K: int
    group_size: int
    # lazily created split-K workspaces (uint8), one per stream the weight is used on: calls that share a workspace
    # must not overlap in time, and work on one stream does not
    workspaces: dict = dataclasses.field(default_factory=dict)

    @property
    def device(self):
        return self.w_r.device

    @property
    def workspace(self) -> Optional[torch.Tensor]:
        """The workspace of the current stream (None if no call on it has needed one yet)."""
        return self.workspaces.get(_stream_ptr(self.device))


@dataclasses.dataclass
class QuantizedActivation:
    q: torch.Tensor        # int8 [M, K]
    s_a: torch.Tensor      # float32 [M]
    rowsum: Optional[torch.Tensor]   # int32 [G, ldr]; None: quantised without group sums (tiled kernel, symmetric levels)
    group_size: int


def repack_w2(packed, scales, zp=None, group_size: int = 128, zp_const: int = 2,
              device="cuda") -> W2A8Weight:
    """Interchange format -> streaming layout, on the GPU.

    packed: uint8 [N, K/4] (pack_matrix layout), scales: float16 [G, N] (quantize layout),
    zp: uint8 [G, N] or None for a uniform zero-point ``zp_const``.  numpy arrays or tensors."""
    L = _lib.lib()
    dev = torch.device(device)
    def host(a):  # torch wants writable memory under a tensor: a read-only array (a mapped file) is copied
        if not isinstance(a, np.ndarray):
            return a
        a = np.ascontiguousarray(a)
        return a if a.flags.writeable else a.copy()
    packed_t = torch.as_tensor(host(packed))
    scales_t = torch.as_tensor(host(scales))
    if packed_t.dtype != torch.uint8 or packed_t.dim() != 2:
        raise ValueError("packed must be a 2-D uint8 array [N, K/4]")
    if scales_t.dtype != torch.float16 or scales_t.dim() != 2:
        raise ValueError("scales must be a 2-D float16 array [G, N]")
    N, K = packed_t.shape[0], packed_t.shape[1] * 4
    if K % group_size != 0 or tuple(scales_t.shape) != (K // group_size, N):
        raise ValueError(f"scales shape {tuple(scales_t.shape)} does not match (K/group_size, N) = "
                         f"{(K // group_size if group_size else 0, N)}")
    packed_d = packed_t.to(dev).contiguous()
    scales_d = scales_t.to(dev).contiguous()
    zp_d = None
    if zp is not None:
        zp_t = torch.as_tensor(host(zp))
        if zp_t.dtype != torch.uint8 or tuple(zp_t.shape) != tuple(scales_t.shape):
            raise ValueError("zp must be uint8 with the shape of scales")
        zp_d = zp_t.to(dev).contiguous()
    wb = L.slimk_w2a8_repacked_weight_bytes(N, K)
    sb = L.slimk_w2a8_repacked_scale_bytes(N, K, group_size)
    if wb == 0 or sb == 0:
        raise ValueError(f"unsupported shape N={N}, K={K}, group_size={group_size} "
                         "(K % 64 == 0, group_size in (64, 128, 256), K % group_size == 0)")
    w_r = torch.empty(wb // 4, dtype=torch.int32, device=dev)
    s_r = torch.empty(sb // 2, dtype=torch.float16, device=dev)
    zp_r = torch.empty(L.slimk_w2a8_repacked_zp_bytes(N, K, group_size), dtype=torch.uint8, device=dev) \
        if zp_d is not None else None
    with torch.cuda.device(dev):
        _lib.check(L.slimk_w2a8_repack(packed_d.data_ptr(), packed_d.stride(0), scales_d.data_ptr(),
                                       zp_d.data_ptr() if zp_d is not None else None, N, K, group_size,
                                       w_r.data_ptr(), s_r.data_ptr(),
                                       zp_r.data_ptr() if zp_r is not None else None, _stream_ptr(dev)))
        # packed_d / scales_d are consumed by the enqueued kernels: keep them alive until done
        torch.cuda.current_stream(dev).synchronize()
    return W2A8Weight(w_r, s_r, zp_r, int(zp_const), N, K, group_size)


def quantize_weight_gpu(weight_nk: torch.Tensor, group_size: int = 128, mode: str = "sym"):
    """Group-wise 2-bit quantisation of an fp16 / bf16 weight [N, K] on the GPU: the same numbers as
    ``slimkernels_amd.prepare_w2`` on the host.  Returns (packed uint8 [N, K/4], scales float16 [G, N],
    zero-points uint8 [G, N]) as device tensors in the interchange layout."""
    L = _lib.lib()
    _require_cuda(weight_nk, "weight")
    if weight_nk.dim() != 2 or weight_nk.dtype not in _DT:
        raise ValueError("weight must be a 2-D float16 or bfloat16 tensor [N, K]")
    modes = {"ref": _lib.QUANT_REF, "sym": _lib.QUANT_SYM, "asym": _lib.QUANT_ASYM}
    if mode not in modes:
        raise ValueError(f"unknown quantizer mode {mode!r} (expected 'ref', 'sym' or 'asym')")
    w = weight_nk if weight_nk.stride(1) == 1 and weight_nk.stride(0) % 8 == 0 and weight_nk.data_ptr() % 16 == 0 \
        else weight_nk.contiguous()
    N, K = w.shape
    if group_size not in (64, 128, 256) or K % group_size != 0:
        raise ValueError(f"unsupported K={K}, group_size={group_size} (group_size in (64, 128, 256), K % group_size == 0)")
    dev = w.device
    packed = torch.empty((N, K // 4), dtype=torch.uint8, device=dev)
    scales = torch.empty((K // group_size, N), dtype=torch.float16, device=dev)
    zero = torch.empty((K // group_size, N), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _lib.check(L.slimk_w2a8_quantize_weight(w.data_ptr(), w.stride(0), _DT[w.dtype], N, K, group_size, modes[mode],
                                                packed.data_ptr(), packed.stride(0), scales.data_ptr(), zero.data_ptr(),
                                                _stream_ptr(dev)))
        if w is not weight_nk:
            torch.cuda.current_stream(dev).synchronize()  # the contiguous copy is consumed by the enqueued kernel
    return packed, scales, zero


def load_w2_weight(path, device="cuda", mmap=True) -> W2A8Weight:
    """Read a weight file written by ``slimkernels_amd.packed_format.save_w2`` (the interchange
    layout) and re-lay it for the GPU: the streaming layout exists only in device memory."""
    from ..packed_format import load_w2
    f = load_w2(path, mmap=mmap)
    return repack_w2(np.ascontiguousarray(f["packed"]), np.ascontiguousarray(f["scales"]), f["zp"], f["group_size"],
                     zp_const=f["zp_const"] if f["zp_const"] is not None else 0, device=device)


def quantize_act_int8(x: torch.Tensor, group_size: int = 128, copies: int = 1, rowsum: bool = True) -> QuantizedActivation:
    """Per-token symmetric int8 quantisation: x [M, K] fp16/bf16 -> q, s_a, per-group row sums.  With
    ``copies`` > 1 the quantised row and its group sums are laid down that many times (q [M, copies * K],
    rowsum [copies * G, ...]): the operand of a reduction over copies * K, as the 4-bit weights take it.
    ``rowsum=False`` leaves the group sums out (faster on many rows); only the tiled kernel on weights with the
    symmetric levels takes such an activation (see ``needs_rowsum``)."""
    L = _lib.lib()
    _require_cuda(x, "x")
    if x.dim() != 2 or x.dtype not in _DT:
        raise ValueError("x must be a 2-D float16 or bfloat16 tensor")
    M, K = x.shape
    if x.stride(1) != 1 or x.stride(0) % 8 != 0 or x.stride(0) < K or x.data_ptr() % 16 != 0:
        x = x.contiguous()
        if x.data_ptr() % 16 != 0:      # contiguous already, but not at a 16-byte boundary
            x = x.clone()
    ldr = (M + 3) // 4 * 4
    copies = int(copies)
    q = torch.empty((M, max(copies, 1) * K), dtype=torch.int8, device=x.device)
    s_a = torch.empty((M,), dtype=torch.float32, device=x.device)
    rs = torch.empty((max(copies, 1) * max(K // group_size, 1), ldr), dtype=torch.int32, device=x.device) if rowsum else None
    with torch.cuda.device(x.device):
        _lib.check(L.slimk_w2a8_act_quant_rep(x.data_ptr(), x.stride(0), _DT[x.dtype], M, K, group_size, copies,
                                              q.data_ptr(), q.stride(0), s_a.data_ptr(),
                                              rs.data_ptr() if rs is not None else None, ldr, _stream_ptr(x.device)))
    return QuantizedActivation(q, s_a, rs, group_size)


def needs_rowsum(M: int, w: "W2A8Weight") -> bool:
    """Whether ``w2a8_gemm(..., kernel="auto")`` of M token rows on this weight reads the activation's group sums:
    everything but the tiled kernel and the kernel for 33..128 rows on the symmetric levels (uniform zero-point 2) does."""
    if w.zp_r is not None or w.zp_const != 2 or w.group_size > 256:
        return True
    return _lib.lib().slimk_w2a8_gemm_auto_route(M, w.N, w.K, w.group_size) not in (2, 4)


def _workspace(w: W2A8Weight, nbytes: int) -> Optional[torch.Tensor]:
    if nbytes == 0:
        return None
    key = _stream_ptr(w.device)
    ws = w.workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
        # only the arrival counters at its start have to be zero; the partial tiles are written before they are read
        _lib.check(_lib.lib().slimk_w2a8_workspace_init(ws.data_ptr(), min(ws.numel(), _lib.COUNTER_BLOCK_BYTES), key))
        w.workspaces[key] = ws
    return ws


def w2a8_gemm(qa: QuantizedActivation, w: W2A8Weight, out_dtype=torch.float16, *, kernel: str = "auto",
              split_k: int = 0, dump: Optional[str] = None, out: Optional[torch.Tensor] = None):
    """out[M, N] = dequant( q @ (codes - zp)^T ).  Returns out, or (out, acc) when ``dump`` is
    "groups" (int32 [M, N, G]) or "sum" (int32 [M, N])."""
    L = _lib.lib()
    kern = {"auto": _lib.KERNEL_AUTO, "skinny": _lib.KERNEL_SKINNY, "tiled": _lib.KERNEL_TILED, "mid": _lib.KERNEL_MID}[kernel]
    M, K = qa.q.shape
    if K != w.K or qa.group_size != w.group_size:
        raise ValueError(f"activation K={K}/group {qa.group_size} does not match weight K={w.K}/group {w.group_size}")
    if out_dtype not in _DT:
        raise ValueError("out_dtype must be torch.float16 or torch.bfloat16")
    dev = qa.q.device
    if out is None:
        out = torch.empty((M, w.N), dtype=out_dtype, device=dev)
    G = K // w.group_size
    acc, mode = None, _lib.DUMP_NONE
    if dump == "groups":
        acc, mode = torch.empty((M, w.N, G), dtype=torch.int32, device=dev), _lib.DUMP_GROUPS
    elif dump == "sum":
        acc, mode = torch.empty((M, w.N), dtype=torch.int32, device=dev), _lib.DUMP_SUM
    elif dump is not None:
        raise ValueError("dump must be None, 'groups' or 'sum'")
    with torch.cuda.device(dev):
        ws_bytes = L.slimk_w2a8_gemm_workspace_bytes(M, w.N, K, w.group_size, kern, split_k)
        ws = _workspace(w, ws_bytes)
        _lib.check(L.slimk_w2a8_gemm(
            qa.q.data_ptr(), qa.q.stride(0), qa.s_a.data_ptr(),
            qa.rowsum.data_ptr() if qa.rowsum is not None else None,
            qa.rowsum.stride(0) if qa.rowsum is not None else (M + 3) // 4 * 4,
            w.w_r.data_ptr(), w.s_r.data_ptr(), w.zp_r.data_ptr() if w.zp_r is not None else None, w.zp_const,
            M, w.N, K, w.group_size, out.data_ptr(), out.stride(0), _DT[out.dtype],
            acc.data_ptr() if acc is not None else None, mode,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
            kern, split_k, _stream_ptr(dev)))
    return (out, acc) if acc is not None else out


FUSED_MAX_ROWS = 32
FUSED_IN_WORKGROUP_ROWS, FUSED_IN_WORKGROUP_BYTES = 4, 32768


def fused_applies(M: int, K: int) -> bool:
    """Whether w2a8_linear_fused takes this shape: up to 32 token rows (up to four rows of at most 32 KiB of int8
    values together are quantised by every workgroup for itself, more or longer rows by the grid's first workgroups
    into the workspace)."""
    return 1 <= M <= FUSED_MAX_ROWS


def w2a8_linear_fused(x: torch.Tensor, w: W2A8Weight, out_dtype=torch.float16, *, split_k: int = 0,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[M, N] for up to 32 token rows x [M, K] fp16 / bf16 in ONE launch: the activation
    quantisation runs inside the GEMM kernel.  Bit-identical with
    ``w2a8_gemm(quantize_act_int8(x), w, kernel="skinny", split_k=...)`` on the one-strip-per-workgroup kernel."""
    L = _lib.lib()
    _require_cuda(x, "x")
    if x.dim() != 2 or x.dtype not in _DT:
        raise ValueError("x must be a 2-D float16 or bfloat16 tensor [M, K]")
    if out_dtype not in _DT:
        raise ValueError("out_dtype must be torch.float16 or torch.bfloat16")
    M, K = x.shape
    if K != w.K:
        raise ValueError(f"activation K={K} does not match weight K={w.K}")
    if not fused_applies(M, K):
        raise ValueError(f"w2a8_linear_fused handles 1 <= M <= {FUSED_MAX_ROWS} (M={M})")
    if x.stride(1) != 1 or x.stride(0) % 8 != 0 or x.stride(0) < K or x.data_ptr() % 16 != 0:
        x = x.contiguous()
        if x.data_ptr() % 16 != 0:      # contiguous already, but not at a 16-byte boundary
            x = x.clone()
    dev = x.device
    if out is None:
        out = torch.empty((M, w.N), dtype=out_dtype, device=dev)
    with torch.cuda.device(dev):
        ws_bytes = L.slimk_w2a8_gemm_fused_workspace_bytes(M, w.N, K, w.group_size, split_k)
        ws = _workspace(w, ws_bytes)
        _lib.check(L.slimk_w2a8_gemm_fused(
            x.data_ptr(), x.stride(0), _DT[x.dtype], w.w_r.data_ptr(), w.s_r.data_ptr(),
            w.zp_r.data_ptr() if w.zp_r is not None else None, w.zp_const, M, w.N, K, w.group_size,
            out.data_ptr(), out.stride(0), _DT[out.dtype],
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, split_k, _stream_ptr(dev)))
    return out


def w2a16_gemm(x: torch.Tensor, w: W2A8Weight, out_dtype=torch.float16, *, split_k: int = 0,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The weight-only form: out[M, N] = x @ dequant(W)^T with the fp16 or bf16 activations x [M, K] as they are (no
    activation quantisation), the 2-bit codes widened in front of the fp16 resp. bf16 matrix cores, fp32 sums.
    Built for few token rows; K must be a multiple of 128."""
    L = _lib.lib()
    _require_cuda(x, "x")
    if x.dim() != 2 or x.dtype not in _DT:
        raise ValueError("x must be a 2-D float16 or bfloat16 tensor [M, K]")
    if out_dtype not in _DT:
        raise ValueError("out_dtype must be torch.float16 or torch.bfloat16")
    M, K = x.shape
    if K != w.K:
        raise ValueError(f"activation K={K} does not match weight K={w.K}")
    if x.stride(1) != 1 or x.stride(0) % 8 != 0 or x.stride(0) < K or x.data_ptr() % 16 != 0:
        x = x.contiguous()
        if x.data_ptr() % 16 != 0:      # contiguous already, but not at a 16-byte boundary
            x = x.clone()
    dev = x.device
    if out is None:
        out = torch.empty((M, w.N), dtype=out_dtype, device=dev)
    with torch.cuda.device(dev):
        ws_bytes = L.slimk_w2a16_gemm_workspace_bytes(M, w.N, K, w.group_size, split_k)
        ws = getattr(w, "_partials16", None)      # its own buffer: the W2A8 workspace holds counters that must stay zero
        if ws_bytes and (ws is None or ws.numel() < ws_bytes):
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            w._partials16 = ws
        _lib.check(L.slimk_w2a16_gemm(
            x.data_ptr(), x.stride(0), _DT[x.dtype], w.w_r.data_ptr(), w.s_r.data_ptr(),
            w.zp_r.data_ptr() if w.zp_r is not None else None, w.zp_const, M, w.N, K, w.group_size,
            out.data_ptr(), out.stride(0), _DT[out.dtype],
            ws.data_ptr() if ws_bytes else None, ws.numel() if ws_bytes else 0, split_k, _stream_ptr(dev)))
    return out


def w2a16_gemm_grouped(problems, out_dtype=torch.float16):
    """Several independent weight-only GEMMs in one kernel launch.

    ``problems`` is a sequence of (x, W2A8Weight) or (x, w, out) tuples whose activations share one type (float16 or
    bfloat16) and whose weights share group size and zero-point mode; returns the list of outputs.  More than 24
    problems are issued as several launches."""
    L = _lib.lib()
    probs = [(p[0], p[1], p[2] if len(p) > 2 else None) for p in problems]
    if not probs:
        return []
    dev = probs[0][0].device
    xdt = probs[0][0].dtype
    g = probs[0][1].group_size
    if xdt not in _DT or out_dtype not in _DT:
        raise ValueError("activations and out_dtype must be torch.float16 or torch.bfloat16")
    outs, keep = [], []
    with torch.cuda.device(dev):
        for lo in range(0, len(probs), _lib.MAX_GROUP):
            chunk = probs[lo:lo + _lib.MAX_GROUP]
            arr = (_lib.Problem16 * len(chunk))()
            for i, (x, w, out) in enumerate(chunk):
                _require_cuda(x, "x")
                if x.dim() != 2 or x.dtype != xdt or x.shape[1] != w.K or w.group_size != g:
                    raise ValueError("grouped problems must share the activation type and group size and match their weights' K")
                M, K = x.shape
                if x.stride(1) != 1 or x.stride(0) % 8 != 0 or x.stride(0) < K or x.data_ptr() % 16 != 0:
                    x = x.contiguous()
                    if x.data_ptr() % 16 != 0:
                        x = x.clone()
                keep.append(x)
                if out is None:
                    out = torch.empty((M, w.N), dtype=out_dtype, device=dev)
                if out.dtype != out_dtype:
                    raise ValueError("every output must have dtype out_dtype")
                outs.append(out)
                arr[i] = _lib.Problem16(x.data_ptr(), w.w_r.data_ptr(), w.s_r.data_ptr(),
                                        w.zp_r.data_ptr() if w.zp_r is not None else None, out.data_ptr(),
                                        x.stride(0), out.stride(0), M, w.N, K, w.zp_const)
            _lib.check(L.slimk_w2a16_gemm_grouped(ctypes.byref(arr), len(chunk), g, _DT[xdt], _DT[out_dtype], _stream_ptr(dev)))
    return outs


def w2a8_gemm_grouped(problems, out_dtype=torch.float16, *, dump: Optional[str] = None):
    """Several independent skinny (M <= 32) GEMMs in one kernel launch.

    ``problems`` is a sequence of (QuantizedActivation, W2A8Weight) or (qa, w, out) tuples that
    share group size and zero-point mode; returns the list of outputs.  More than 24 problems are
    issued as several launches.  With ``dump`` ("groups" or "sum") the verification instantiation of
    the grouped kernel runs and (outputs, int32 accumulator tensors) is returned."""
    L = _lib.lib()
    probs = [(p[0], p[1], p[2] if len(p) > 2 else None) for p in problems]
    if not probs:
        return []
    dev = probs[0][0].q.device
    g = probs[0][1].group_size
    if dump not in (None, "groups", "sum"):
        raise ValueError("dump must be None, 'groups' or 'sum'")
    outs, accs = [], []
    with torch.cuda.device(dev):
        for lo in range(0, len(probs), _lib.MAX_GROUP):
            chunk = probs[lo:lo + _lib.MAX_GROUP]
            arr = (_lib.Problem * len(chunk))()
            dumps = (ctypes.c_void_p * len(chunk))()
            for i, (qa, w, out) in enumerate(chunk):
                M, K = qa.q.shape
                if K != w.K or qa.group_size != w.group_size or w.group_size != g:
                    raise ValueError("grouped problems must share the group size and match their weights' K")
                if out is None:
                    out = torch.empty((M, w.N), dtype=out_dtype, device=dev)
                if out.dtype != out_dtype:
                    raise ValueError("every output must have dtype out_dtype")
                outs.append(out)
                if dump is not None:
                    shape = (M, w.N, K // g) if dump == "groups" else (M, w.N)
                    accs.append(torch.empty(shape, dtype=torch.int32, device=dev))
                    dumps[i] = accs[-1].data_ptr()
                arr[i] = _lib.Problem(qa.q.data_ptr(), qa.s_a.data_ptr(), qa.rowsum.data_ptr(), w.w_r.data_ptr(),
                                      w.s_r.data_ptr(), w.zp_r.data_ptr() if w.zp_r is not None else None,
                                      out.data_ptr(), qa.q.stride(0), qa.rowsum.stride(0), out.stride(0),
                                      M, w.N, K, w.zp_const)
            if dump is None:
                _lib.check(L.slimk_w2a8_gemm_grouped(ctypes.byref(arr), len(chunk), g, _DT[out_dtype], _stream_ptr(dev)))
            else:
                _lib.check(L.slimk_w2a8_gemm_grouped_verify(
                    ctypes.byref(arr), len(chunk), g, _DT[out_dtype], ctypes.byref(dumps),
                    _lib.DUMP_GROUPS if dump == "groups" else _lib.DUMP_SUM, _stream_ptr(dev)))
    return outs if dump is None else (outs, accs)


def wint2_gemm(activation: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor, zp=None,
               group_size: Optional[int] = None, zp_const: int = 2, out_dtype=None) -> torch.Tensor:
    """One-shot form with the argument order of the upstream notebook entry
    wint2_gemm(activation, weight, scale) (triton.ipynb cell 1): ``activation`` [M, K]
    fp16/bf16, ``weight`` the packed matrix transposed, [K/4, N] uint8 (upstream passes
    ``packed_weight.T``), ``scale`` [G, N] fp16.  The weight is re-laid for the GPU on the first call with
    a given (weight, scale, zp) and kept for the next ones (a handful of layers; tensors are recognised by
    identity and version counter, so an in-place change re-lays them; numpy arrays are re-laid every time)."""
    _require_cuda(activation, "activation")
    K = weight.shape[0] * 4
    if group_size is None:
        group_size = K // scale.shape[0]
    w = _wint2_weight(weight, scale, zp, group_size, zp_const, activation.device)
    qa = quantize_act_int8(activation, group_size)
    return w2a8_gemm(qa, w, out_dtype or activation.dtype)


_WINT2_CACHE: "collections.OrderedDict" = collections.OrderedDict()
_WINT2_CACHE_SIZE = 16


def _wint2_weight(weight, scale, zp, group_size, zp_const, device) -> W2A8Weight:
    """The repacked form of wint2_gemm's weight operands, cached by tensor identity and version."""
    tensors = [t for t in (weight, scale, zp) if t is not None]
    if not all(isinstance(t, torch.Tensor) for t in tensors):
        return repack_w2(np.ascontiguousarray(np.asarray(weight).T) if not isinstance(weight, torch.Tensor) else weight.t().contiguous(),
                         scale, zp, group_size, zp_const, device=device)
    # A tensor is recognised by the memory it views (storage address, offset, shape, strides, dtype) and its version
    # counter, not by the Python object: `packed.T` makes a new view object on every call.  The version counter cannot
    # be read on inference-mode tensors: such operands are re-laid every call instead of failing.
    try:
        key = tuple((t.untyped_storage().data_ptr(), t.storage_offset(), tuple(t.shape), tuple(t.stride()), t.dtype,
                     t._version) for t in tensors) + (zp is None, group_size, zp_const, str(device))
    except RuntimeError:
        return repack_w2(weight.t().contiguous(), scale, zp, group_size, zp_const, device=device)
    hit = _WINT2_CACHE.get(key)
    if hit is not None:
        _WINT2_CACHE.move_to_end(key)
        return hit[0]
    w = repack_w2(weight.t().contiguous(), scale, zp, group_size, zp_const, device=device)
    # the storages are held (not the views) so that their addresses stay theirs while the entry lives
    _WINT2_CACHE[key] = (w, [t.untyped_storage() for t in tensors])
    while len(_WINT2_CACHE) > _WINT2_CACHE_SIZE:
        _WINT2_CACHE.popitem(last=False)
    return w


class W2A8Linear(torch.nn.Module):
    """y = x @ W^T with W held as 2-bit codes (+ optional bias), a swap-in for nn.Linear."""

    def __init__(self, weight: W2A8Weight, bias: Optional[torch.Tensor] = None, out_dtype=torch.float16):
        super().__init__()
        self.weight = weight
        self.bias = bias
        self.out_dtype = out_dtype
        self.in_features, self.out_features = weight.K, weight.N

    @classmethod
    def from_float(cls, weight_nk, group_size=128, mode="sym", bias=None, out_dtype=torch.float16, device="cuda"):
        from ..quantization import prepare_w2
        uniform = {"sym": 2, "ref": 1}.get(mode)
        if isinstance(weight_nk, torch.Tensor) and weight_nk.is_cuda and weight_nk.dtype in _DT:
            # quantise where the weight already is (same numbers as the host path)
            packed, scales, zero = quantize_weight_gpu(weight_nk.detach(), group_size, mode)
            w = repack_w2(packed, scales, None if uniform is not None else zero, group_size,
                          zp_const=uniform if uniform is not None else 0, device=weight_nk.device)
            return cls(w, bias, out_dtype)
        w_np = weight_nk.detach().float().cpu().numpy() if isinstance(weight_nk, torch.Tensor) else np.asarray(weight_nk)
        packed, scales, zero = prepare_w2(w_np, group_size, mode)
        w = repack_w2(packed, scales, None if uniform is not None else zero, group_size,
                      zp_const=uniform if uniform is not None else 0, device=device)
        return cls(w, bias, out_dtype)

    @classmethod
    def from_file(cls, path, bias=None, out_dtype=torch.float16, device="cuda"):
        """A layer from a packed weight file (slimkernels_amd.packed_format)."""
        return cls(load_w2_weight(path, device), bias, out_dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        if x2.dtype not in _DT:
            x2 = x2.to(self.out_dtype)
        if x2.shape[0] == 1 and fused_applies(1, x2.shape[1]):
            # one token row: one launch with the quantisation inside the GEMM (measured 6.1 us against 8.0 us at
            # 4096 x 4096; from two rows on the separate act-quant launch is as fast or faster)
            y = w2a8_linear_fused(x2, self.weight, self.out_dtype)
        else:
            # prefill-sized inputs on symmetric weights go to the tiled kernel, which reads no group sums: leave them out
            qa = quantize_act_int8(x2, self.weight.group_size, rowsum=needs_rowsum(x2.shape[0], self.weight))
            y = w2a8_gemm(qa, self.weight, self.out_dtype)
        if self.bias is not None:
            y = y + self.bias
        return y.reshape(*lead, self.out_features)


class W2A16Linear(W2A8Linear):
    """The same layer with the activations left in fp16 or bf16 (weight-only quantisation): forward runs the
    weight-only kernel, meant for a few token rows; the weight object and the constructors are W2A8Linear's."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        if x2.dtype not in _DT:
            x2 = x2.to(torch.float16)
        y = w2a16_gemm(x2, self.weight, self.out_dtype)
        if self.bias is not None:
            y = y + self.bias
        return y.reshape(*lead, self.out_features)
