"""CPU oracle for the W2A8 GEMM path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this
module; the product package (slimkernels_amd) never does.

Two independent restatements live here so that each pins the other:

* the scalar C library ``libw2a8_oracle.so`` (built from w2a8_oracle.c by
  oracle/Makefile), wrapped by the ``c_*`` functions;
* vectorised numpy versions (``np_*``) of the same closed forms, plus an
  exact-in-floating-point BLAS form of the integer GEMM for shapes the scalar
  loop would take minutes on.

Reference anchors (upstream SlimKernels tree):
  pack / unpack     matrix_packer.py:29-34, :57-64
  REF quantizer     quantization.py:26-46   (zero_point 1, absmax/1.5, np.round)
  dequantizer       quantization.py:83-93
The int8 activation quantizer, int32 accumulation and epilogue have no upstream
counterpart; tests/test_oracle.py pins them by brute force and exact identities.
The weight-only form (w2a16_reference_forward; upstream's sketch is the notebook kernel
w2matmul, gemm_splitk.ipynb cell 1, which has no test and no stored output) is parity
unpinned against upstream; tests/test_w2a16.py pins it by a hand case, torch's float64
matmul on the dequantised weight and plain loops.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libw2a8_oracle.so")

MODE_REF, MODE_SYM, MODE_ASYM = 0, 1, 2
_MODES = {"ref": MODE_REF, "sym": MODE_SYM, "asym": MODE_ASYM}


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (seconds).  Returns the library path."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "w2a8_oracle.c"))
    ):
        subprocess.run(["make", "-C", _HERE, "-B", "libw2a8_oracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        c_long, c_int, vp = ctypes.c_long, ctypes.c_int, ctypes.c_void_p
        L.w2o_pack.argtypes = [vp, c_long, c_long, vp]
        L.w2o_unpack.argtypes = [vp, c_long, c_long, vp]
        L.w2o_quantize_w2.argtypes = [vp, c_long, c_long, c_long, c_int, vp, vp, vp]
        L.w2o_dequantize_w2.argtypes = [vp, vp, vp, c_long, c_long, c_long, vp]
        L.w2o_act_quant.argtypes = [vp, c_int, c_long, c_long, c_long, vp, vp, vp, c_long]
        L.w2o_gemm_acc.argtypes = [vp, vp, vp, c_long, c_long, c_long, c_long, vp]
        L.w2o_epilogue.argtypes = [vp, vp, vp, c_long, c_long, c_long, c_int, vp, vp]
        L.w2o_gemm_fused.argtypes = [vp, vp, vp, vp, vp, c_long, c_long, c_long, c_long, c_int, vp, vp]
        L.w2o_half_to_float.argtypes = [ctypes.c_uint16]
        L.w2o_half_to_float.restype = ctypes.c_float
        L.w2o_float_to_half.argtypes = [ctypes.c_float]
        L.w2o_float_to_half.restype = ctypes.c_uint16
        L.w2o_float_to_bf16.argtypes = [ctypes.c_float]
        L.w2o_float_to_bf16.restype = ctypes.c_uint16
        L.w2o_bf16_to_float.argtypes = [ctypes.c_uint16]
        L.w2o_bf16_to_float.restype = ctypes.c_float
        _lib = L
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


# --------------------------------------------------------------------------- C wrappers

def c_pack(codes: np.ndarray) -> np.ndarray:
    codes = _c(codes, np.uint8)
    rows, cols = codes.shape
    out = np.empty((rows, max(cols // 4, 0)), np.uint8)
    rc = lib().w2o_pack(_p(codes), rows, cols, _p(out))
    if rc:
        raise ValueError(f"w2o_pack rc={rc}")
    return out


def c_unpack(packed: np.ndarray) -> np.ndarray:
    packed = _c(packed, np.uint8)
    rows, pc = packed.shape
    out = np.empty((rows, pc * 4), np.uint8)
    lib().w2o_unpack(_p(packed), rows, pc, _p(out))
    return out


def c_quantize_w2(w_kn: np.ndarray, group_size: int, mode: str):
    """w_kn [K, N] -> codes uint8 [K, N], scales float32 [G, N], zp uint8 [G, N]."""
    w = _c(w_kn, np.float32)
    K, N = w.shape
    G = K // group_size
    codes = np.empty((K, N), np.uint8)
    scales = np.empty((G, N), np.float32)
    zp = np.empty((G, N), np.uint8)
    rc = lib().w2o_quantize_w2(_p(w), K, N, group_size, _MODES[mode], _p(codes), _p(scales), _p(zp))
    if rc:
        raise ValueError(f"w2o_quantize_w2 rc={rc}")
    return codes, scales, zp


def c_dequantize_w2(codes, scales, zp, group_size: int) -> np.ndarray:
    codes = _c(codes, np.uint8)
    K, N = codes.shape
    out = np.empty((K, N), np.float16)
    rc = lib().w2o_dequantize_w2(_p(codes), _p(_c(scales, np.float32)), _p(_c(zp, np.uint8)),
                                 K, N, group_size, _p(out))
    if rc:
        raise ValueError(f"w2o_dequantize_w2 rc={rc}")
    return out


def c_act_quant(x_bits: np.ndarray, group_size: int, is_bf16: bool = False):
    """x_bits: [M, K] float16 array, or uint16 holding bf16 bits when is_bf16.
    Returns q int8 [M, K], s_a float32 [M], rowsum int32 [G, M]."""
    xb = np.ascontiguousarray(x_bits).view(np.uint16)
    M, K = xb.shape
    G = K // group_size
    q = np.empty((M, K), np.int8)
    s_a = np.empty((M,), np.float32)
    rs = np.empty((G, M), np.int32)
    rc = lib().w2o_act_quant(_p(xb), int(is_bf16), M, K, group_size, _p(q), _p(s_a), _p(rs), M)
    if rc:
        raise ValueError(f"w2o_act_quant rc={rc}")
    return q, s_a, rs


def c_gemm_acc(q, packed, zp, group_size: int) -> np.ndarray:
    """acc int32 [M, N, G]."""
    q = _c(q, np.int8)
    packed = _c(packed, np.uint8)
    zp = _c(zp, np.uint8)
    M, K = q.shape
    N = packed.shape[0]
    G = K // group_size
    acc = np.empty((M, N, G), np.int32)
    rc = lib().w2o_gemm_acc(_p(q), _p(packed), _p(zp), M, N, K, group_size, _p(acc))
    if rc:
        raise ValueError(f"w2o_gemm_acc rc={rc}")
    return acc


def c_epilogue(acc, scale_half, s_a, out_bf16: bool = False):
    """Returns (out_bits uint16 [M, N] (fp16 or bf16 bit patterns), out_f32 [M, N])."""
    acc = _c(acc, np.int32)
    M, N, G = acc.shape
    sh = _c(scale_half, np.float16)
    out = np.empty((M, N), np.uint16)
    of = np.empty((M, N), np.float32)
    lib().w2o_epilogue(_p(acc), _p(sh), _p(_c(s_a, np.float32)), M, N, G, int(out_bf16), _p(out), _p(of))
    return out, of


def c_gemm_fused(q, s_a, packed, scale_half, zp, group_size: int, out_bf16: bool = False,
                 want_acc_sum: bool = False):
    q = _c(q, np.int8)
    packed = _c(packed, np.uint8)
    M, K = q.shape
    N = packed.shape[0]
    out = np.empty((M, N), np.uint16)
    acc_sum = np.empty((M, N), np.int32) if want_acc_sum else None
    rc = lib().w2o_gemm_fused(_p(q), _p(_c(s_a, np.float32)), _p(packed), _p(_c(scale_half, np.float16)),
                              _p(_c(zp, np.uint8)), M, N, K, group_size, int(out_bf16), _p(out),
                              _p(acc_sum) if want_acc_sum else None)
    if rc:
        raise ValueError(f"w2o_gemm_fused rc={rc}")
    return out, acc_sum


# --------------------------------------------------------------------------- numpy restatements

def np_pack(codes: np.ndarray) -> np.ndarray:
    """matrix_packer.py:33-34 as one vector expression."""
    c = np.asarray(codes, np.uint8)
    c4 = c.reshape(c.shape[0], -1, 4).astype(np.uint16)
    return ((c4[..., 0] << 6) | (c4[..., 1] << 4) | (c4[..., 2] << 2) | c4[..., 3]).astype(np.uint8)


def np_unpack(packed: np.ndarray) -> np.ndarray:
    """matrix_packer.py:61-64."""
    b = np.asarray(packed, np.uint8)
    out = np.stack([(b >> 6) & 3, (b >> 4) & 3, (b >> 2) & 3, b & 3], axis=-1)
    return out.reshape(b.shape[0], -1).astype(np.uint8)


def np_quantize_w2(w_kn: np.ndarray, group_size: int, mode: str):
    w = np.asarray(w_kn, np.float32)
    K, N = w.shape
    G = K // group_size
    r = w.reshape(G, group_size, N)
    one = np.float32
    if mode == "ref":
        s = np.maximum(np.abs(r).max(axis=1), one(1e-9)) / one(1.5)
        zp = np.full((G, N), 1, np.float32)
    elif mode == "sym":
        s = np.maximum(np.abs(r).max(axis=1), one(1e-9)) / one(2.0)
        zp = np.full((G, N), 2, np.float32)
    elif mode == "asym":
        mx, mn = r.max(axis=1), r.min(axis=1)
        s = np.maximum(mx - mn, one(1e-9)) / one(3.0)
        zp = np.clip(np.round(-mn / s), 0, 3).astype(np.float32)
    else:
        raise ValueError(mode)
    s = s.astype(np.float32)
    codes = np.clip(np.round(r / s[:, None, :]) + zp[:, None, :], 0, 3).astype(np.uint8)
    return codes.reshape(K, N), s, zp.astype(np.uint8)


def np_act_quant(x: np.ndarray, group_size: int):
    """x float16 [M, K] (or any float array already holding representable values)."""
    xf = np.asarray(x).astype(np.float32)
    M, K = xf.shape
    amax = np.abs(xf).max(axis=1)
    s = (np.maximum(amax, np.float32(1e-9)) / np.float32(127.0)).astype(np.float32)
    q = np.clip(np.round(xf / s[:, None]), -127, 127).astype(np.int8)
    rs = q.astype(np.int32).reshape(M, K // group_size, group_size).sum(axis=2).T.copy()
    return q, s, rs


def np_gemm_acc_blas(q: np.ndarray, codes_nk: np.ndarray, zp_gn: np.ndarray, group_size: int,
                     dtype=np.float64) -> np.ndarray:
    """acc [M, N, G] through a floating-point BLAS matmul per group.

    Every operand is a small integer and every partial sum is bounded by
    g*127*3 < 2**24, so the float result is the exact integer in any summation
    order (float32 and float64 alike)."""
    M, K = q.shape
    N = codes_nk.shape[0]
    G = K // group_size
    acc = np.empty((M, N, G), np.int32)
    qf = q.astype(dtype)
    for gi in range(G):
        ks = slice(gi * group_size, (gi + 1) * group_size)
        w = codes_nk[:, ks].astype(dtype) - zp_gn[gi].astype(dtype)[:, None]
        acc[:, :, gi] = np.rint(qf[:, ks] @ w.T).astype(np.int32)
    return acc


def np_epilogue_f64(acc: np.ndarray, scale_half: np.ndarray, s_a: np.ndarray) -> np.ndarray:
    """Same sum evaluated in float64 (no intermediate rounding worth speaking of):
    the yardstick for the "within 1 ULP of the output type" checks."""
    s = np.asarray(scale_half, np.float16).astype(np.float64)  # [G, N]
    t = np.einsum("mng,gn->mn", acc.astype(np.float64), s)
    return t * np.asarray(s_a, np.float64)[:, None]


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    return ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)


# --------------------------------------------------------------------------- 4-bit weights
# Upstream has no W4 quantiser (gemm_splitk.ipynb cell 0 multiplies by random packed codes); the level
# sets below are this build's: "sym" levels -8..7 with s = absmax / 8, "asym" s = (max - min) / 15.
# Pinned in tests/test_w4a8.py by closed forms, brute force on small inputs and the notebook's
# unpack expression; parity with upstream is unpinned for want of an upstream definition.

def np_pack_w4(codes: np.ndarray) -> np.ndarray:
    """Two codes per byte along the row, first code in the high nibble."""
    c = np.asarray(codes, np.uint8)
    c2 = c.reshape(c.shape[0], -1, 2)
    return ((c2[..., 0] << 4) | c2[..., 1]).astype(np.uint8)


def np_unpack_w4(packed: np.ndarray) -> np.ndarray:
    b = np.asarray(packed, np.uint8)
    return np.stack([b >> 4, b & 15], axis=-1).reshape(b.shape[0], -1).astype(np.uint8)


def np_unpack_uint32_kn(b: np.ndarray) -> np.ndarray:
    """gemm_splitk.ipynb cell 0: code of element k is ``(b[k // 8, n] >> (k % 8) * 4) & 0xF``; returns [N, K]."""
    b = np.asarray(b).astype(np.uint64)
    K = b.shape[0] * 8
    k = np.arange(K)
    return ((b[k // 8, :] >> ((k % 8) * 4)[:, None].astype(np.uint64)) & 15).astype(np.uint8).T.copy()


def np_quantize_w4(w_kn: np.ndarray, group_size: int, mode: str):
    w = np.asarray(w_kn, np.float32)
    K, N = w.shape
    G = K // group_size
    r = w.reshape(G, group_size, N)
    one = np.float32
    if mode == "sym":
        s = np.maximum(np.abs(r).max(axis=1), one(1e-9)) / one(8.0)
        zp = np.full((G, N), 8, np.float32)
    elif mode == "asym":
        mx, mn = r.max(axis=1), r.min(axis=1)
        s = np.maximum(mx - mn, one(1e-9)) / one(15.0)
        zp = np.clip(np.round(-mn / s), 0, 15).astype(np.float32)
    else:
        raise ValueError(mode)
    s = s.astype(np.float32)
    codes = np.clip(np.round(r / s[:, None, :]) + zp[:, None, :], 0, 15).astype(np.uint8)
    return codes.reshape(K, N), s, zp.astype(np.uint8)


def w4_reference_forward(x_half: np.ndarray, codes_nk: np.ndarray, scale_half: np.ndarray, zp: np.ndarray,
                         group_size: int, out_bf16: bool = False):
    """act-quant -> exact int32 per-group sums of q * (code - zp) -> the W2 path's epilogue
    (t = fmaf(float(acc_g), scale[g, n], t) in ascending g, then * s_a, one cast)."""
    q, s_a, rs = c_act_quant(x_half, group_size)
    acc = np_gemm_acc_blas(q, np.asarray(codes_nk, np.uint8), np.asarray(zp, np.uint8), group_size)
    out_bits, out_f32 = c_epilogue(acc, scale_half, s_a, out_bf16)
    return dict(q=q, s_a=s_a, rowsum=rs, acc=acc, out_bits=out_bits, out_f32=out_f32)


def w2a16_reference_forward(x_half: np.ndarray, codes_nk: np.ndarray, scale_half: np.ndarray, zp: np.ndarray,
                            group_size: int, x_bf16: bool = False):
    """The weight-only form in float64: out[m, n] = sum_g scale[g, n] * sum_{k in g} x[m, k] * (code[n, k] - zp[g, n])
    with the fp16 activations as they are (the notebook kernel w2matmul, gemm_splitk.ipynb cell 1, widens the
    2-bit fields to fp16 in front of an fp32-accumulating dot; it has no scales and no zero-point, which are
    this path's own).  Returns (out float64 [M, N], mag float64 [M, N]) where mag = sum_g |scale| * sum_k |x| * |code - zp|
    bounds the terms, for a tolerance on an fp32 accumulation in any order.  With x_bf16 the activations are uint16
    bf16 bit patterns instead of a float16 array."""
    if x_bf16:
        x = (np.asarray(x_half, np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    else:
        x = np.asarray(x_half, np.float16).astype(np.float64)
    codes = np.asarray(codes_nk, np.uint8)
    N, K = codes.shape
    M = x.shape[0]
    G = K // group_size
    w = codes.astype(np.float64).reshape(N, G, group_size) - np.asarray(zp, np.float64).T[:, :, None]
    s = np.asarray(scale_half, np.float16).astype(np.float64).T                       # [N, G]
    xg = x.reshape(M, G, group_size)
    out = np.einsum("mgk,ngk,ng->mn", xg, w, s, optimize=True)
    mag = np.einsum("mgk,ngk,ng->mn", np.abs(xg), np.abs(w), np.abs(s), optimize=True)
    return out, mag


# --------------------------------------------------------------------------- whole-path helper

def reference_forward(x_half: np.ndarray, packed: np.ndarray, scale_half: np.ndarray, zp: np.ndarray,
                      group_size: int, out_bf16: bool = False, want_acc: bool = True, x_bf16: bool = False):
    """act-quant -> int32 per-group accumulate -> epilogue, all on the CPU.  With x_bf16 the activations are
    uint16 bf16 bit patterns instead of a float16 array.

    Returns dict(q, s_a, rowsum, acc (or None), out_bits, out_f32 (or None))."""
    q, s_a, rs = c_act_quant(x_half, group_size, is_bf16=x_bf16)
    if want_acc:
        acc = c_gemm_acc(q, packed, zp, group_size)
        out_bits, out_f32 = c_epilogue(acc, scale_half, s_a, out_bf16)
    else:
        acc, out_f32 = None, None
        out_bits, _ = c_gemm_fused(q, s_a, packed, scale_half, zp, group_size, out_bf16)
    return dict(q=q, s_a=s_a, rowsum=rs, acc=acc, out_bits=out_bits, out_f32=out_f32)


def torch_reference_forward(x_half: np.ndarray, packed: np.ndarray, scale_half: np.ndarray, zp: np.ndarray,
                            group_size: int, out_bf16: bool = False):
    """The CPU path as the task statement words it: numpy quantiser/packer output fed to a
    torch CPU integer matmul, then the float epilogue.  Used for the timed CPU baseline; its
    result agrees with c_gemm_acc exactly (int32) and with c_epilogue to float32 rounding
    (the group sum here is a plain torch sum, not the fused chain)."""
    import torch
    q, s_a, _ = np_act_quant(x_half, group_size)
    M, K = q.shape
    N = packed.shape[0]
    G = K // group_size
    codes = torch.from_numpy(np_unpack(packed)).to(torch.int32).reshape(N, G, group_size)
    w = codes - torch.from_numpy(np.ascontiguousarray(zp.T)).to(torch.int32)[:, :, None]
    acc = torch.einsum("mgk,ngk->mng", torch.from_numpy(q).to(torch.int32).reshape(M, G, group_size), w)
    s = torch.from_numpy(np.ascontiguousarray(np.asarray(scale_half, np.float16).T)).to(torch.float32)  # [N, G]
    t = (acc.to(torch.float32) * s[None]).sum(dim=2) * torch.from_numpy(s_a)[:, None]
    out = t.to(torch.bfloat16 if out_bf16 else torch.float16)
    return acc.numpy(), out
