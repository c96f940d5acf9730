"""Host-side (numpy) definition of the gfx950 streaming weight layout.

The GPU repack kernel (csrc/prep_kernels.hip) is the product path; this module states
the same layout in numpy so that (a) the kernel can be checked bit-for-bit, (b) a
repacked buffer can be turned back into the interchange format (``unrepack_codes``),
e.g. when persisting weights.  Nothing here is used by the GEMM.

Layout: the [N, K] code matrix is cut into units of 64 channels (strip) x 64 reduction
elements (step); unit (step, strip) is 64 lanes x 4 dwords at dword offset
((((step // 4) * strips + strip) * 4 + step % 4) * 64 + lane) * 4: four consecutive steps of a
strip form one run of 4 KiB (what a wave streams back to back), the runs of all strips for the
same four steps follow each other (what all strips read at the same time is one contiguous band);
a step count that is no multiple of four is padded with zero units.  With col = lane & 15, quad = lane >> 4, the
2-bit field p (bits 2p+1:2p) of byte b of dword i holds the code of

    n = strip*64 + p*16 + col        k = step*64 + quad*16 + 4*i + b

and field 3 is stored xor 2 (two's complement of code - 2, it sits in the byte's sign
bits).  Interchange format: matrix_packer.py:33-34 upstream (first code in bits 7:6).
"""
import numpy as np

STRIP_N = 64
STEP_K = 64
RUN_STEPS = 4


def unit(w_r: np.ndarray, step: int, strip: int) -> np.ndarray:
    """The [64 lanes, 4 dwords] unit (step, strip) of a repacked array [runs, strips, 4, 64, 4]."""
    return w_r[step // RUN_STEPS, strip, step % RUN_STEPS]


def repack_codes(packed: np.ndarray) -> np.ndarray:
    """uint8 [N, K/4] interchange bytes -> uint32 [runs, strips, 4, 64, 4] streaming layout (run = four steps)."""
    packed = np.asarray(packed, np.uint8)
    N, K = packed.shape[0], packed.shape[1] * 4
    if K % STEP_K:
        raise ValueError("K must be a multiple of 64")
    strips, steps = -(-N // STRIP_N), K // STEP_K
    shifts = np.array([6, 4, 2, 0], np.uint8)
    codes = ((packed[:, :, None] >> shifts) & 3).reshape(N, K)
    full = np.zeros((strips * STRIP_N, K), np.uint32)
    full[:N] = codes
    # axes: strip, p, col, step, quad, i, b
    c = full.reshape(strips, 4, 16, steps, 4, 4, 4)
    c[:, 3] ^= 2
    out = np.zeros((strips, steps, 4, 16, 4), np.uint32)  # strip, step, quad, col, i
    for p in range(4):
        for b in range(4):
            # c[:, p, :, :, :, :, b] has axes strip, col, step, quad, i
            out |= c[:, p, :, :, :, :, b].transpose(0, 2, 3, 1, 4) << np.uint32(8 * b + 2 * p)
    runs = -(-steps // RUN_STEPS)
    padded = np.zeros((strips, runs * RUN_STEPS, 64, 4), np.uint32)
    padded[:, :steps] = out.reshape(strips, steps, 64, 4)
    return np.ascontiguousarray(padded.reshape(strips, runs, RUN_STEPS, 64, 4).transpose(1, 0, 2, 3, 4))


def unrepack_codes(w_r: np.ndarray, N: int, K: int) -> np.ndarray:
    """Inverse of :func:`repack_codes`: streaming layout -> uint8 [N, K/4] interchange bytes."""
    strips, steps = -(-N // STRIP_N), K // STEP_K
    runs = -(-steps // RUN_STEPS)
    w = np.asarray(w_r, np.uint32).reshape(runs, strips, RUN_STEPS, 64, 4).transpose(1, 0, 2, 3, 4)
    w = w.reshape(strips, runs * RUN_STEPS, 4, 16, 4)[:, :steps]                                # strip, step, quad, col, i
    codes = np.zeros((strips, 4, 16, steps, 4, 4, 4), np.uint8)       # strip, p, col, step, quad, i, b
    for p in range(4):
        for b in range(4):
            f = ((w >> np.uint32(8 * b + 2 * p)) & 3).astype(np.uint8)
            if p == 3:
                f ^= 2
            codes[:, p, :, :, :, :, b] = f.transpose(0, 3, 1, 2, 4)
    codes = codes.reshape(strips * STRIP_N, K)[:N]
    q = codes.reshape(N, K // 4, 4)
    return ((q[..., 0] << 6) | (q[..., 1] << 4) | (q[..., 2] << 2) | q[..., 3]).astype(np.uint8)


def repack_group_values(values_gn: np.ndarray) -> np.ndarray:
    """[G, N] per-(group, channel) values (scales or zero-points) -> [G, strips, 16, 4]
    (group, strip, col, sub-block p), zero-filled past N."""
    v = np.asarray(values_gn)
    G, N = v.shape
    strips = -(-N // STRIP_N)
    full = np.zeros((G, strips * STRIP_N), v.dtype)
    full[:, :N] = v
    return np.ascontiguousarray(full.reshape(G, strips, 4, 16).transpose(0, 1, 3, 2))
