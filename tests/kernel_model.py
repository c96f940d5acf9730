"""numpy model of what one wavefront of the GEMM kernels computes from the streaming
layout (csrc/w2a8_common.h), lane by lane, with the documented operand mapping of
v_mfma_i32_16x16x64_i8:

    A operand: lane l holds row (l & 15), the 16 k-values of quarter (l >> 4)
    B operand: lane l holds col (l & 15), the same 16 k-values
    D        : lane l, element j  ->  row 4*(l >> 4) + j, col (l & 15)

Used by the CPU tests to check the index arithmetic (layout, shift-free unpack, scaled
zero-point folding, group drains) against the oracle without a GPU."""
import numpy as np

MASK = [np.uint32(0x03030303 << (2 * p)) for p in range(4)]


def mfma_16x16x64(a_lanes: np.ndarray, b_lanes: np.ndarray, c_lanes: np.ndarray) -> np.ndarray:
    """a_lanes, b_lanes: int8 [64, 16]; c_lanes: int32 [64, 4] -> d_lanes int32 [64, 4]."""
    A = np.zeros((16, 64), np.int32)
    B = np.zeros((64, 16), np.int32)
    for l in range(64):
        A[l & 15, (l >> 4) * 16:(l >> 4) * 16 + 16] = a_lanes[l]
        B[(l >> 4) * 16:(l >> 4) * 16 + 16, l & 15] = b_lanes[l]
    D = A @ B
    d = c_lanes.copy()
    for l in range(64):
        for j in range(4):
            d[l, j] += D[4 * (l >> 4) + j, l & 15]
    return d


def wave_strip_groups(q, rowsum, w_r, s_r, zp_r, zp_const, strip, groups, gs, M):
    """Model of one wave working through `groups` of one strip for token rows 0..15.
    Returns (t float32 [16, 64], acc int32 [16, 64, len(groups)]) in (m, n_local) order."""
    lanes = np.arange(64)
    col, quad = lanes & 15, lanes >> 4
    t = np.zeros((64, 4, 4), np.float32)  # lane, p, j
    acc_out = np.zeros((16, 64, len(groups)), np.int32)
    for gi, g in enumerate(groups):
        sraw = s_r[g, strip][col]                         # [64, 4] fp16 (lane, p)
        sc = sraw.astype(np.float32) * np.array([1, 0.25, 0.0625, 0.015625], np.float32)
        if zp_r is not None:
            z = zp_r[g, strip][col].astype(np.int32)
        else:
            z = np.full((64, 4), zp_const, np.int32)
        zpe = np.stack([z[:, 0], z[:, 1] * 4, z[:, 2] * 16, (z[:, 3] - 2) * 64], axis=1)
        acc = np.zeros((64, 4, 4), np.int32)
        for l in range(64):
            m0 = quad[l] * 4
            rs = np.array([rowsum[g, m0 + j] if m0 + j < M else 0 for j in range(4)], np.int32)
            for p in range(4):
                acc[l, p] = -zpe[l, p] * rs
        for s in range(gs):
            step = g * gs + s
            w = w_r[step // 4, strip, step % 4]           # uint32 [64, 4]: runs of four steps per strip
            a = np.zeros((64, 16), np.int8)
            for l in range(64):
                m = col[l]
                if m < M:
                    a[l] = q[m, step * 64 + quad[l] * 16: step * 64 + quad[l] * 16 + 16]
            for p in range(4):
                b = (w & MASK[p]).view(np.int8).reshape(64, 16)   # dword i -> bytes 4i..4i+3 (little endian)
                acc[:, p] = mfma_16x16x64(a, b, acc[:, p])
        for l in range(64):
            for p in range(4):
                for j in range(4):
                    t[l, p, j] = np.float32(np.float32(acc[l, p, j]) * sc[l, p] + t[l, p, j])
                    acc_out[quad[l] * 4 + j, p * 16 + col[l], gi] = acc[l, p, j] >> (2 * p)
    tt = np.zeros((16, 64), np.float32)
    for l in range(64):
        for p in range(4):
            for j in range(4):
                tt[quad[l] * 4 + j, p * 16 + col[l]] = t[l, p, j]
    return tt, acc_out
