"""Shared helpers of the GPU parity tests."""
import functools

import numpy as np
import torch

from slimkernels_amd import workloads


def bits_to_f32(bits: np.ndarray, bf16: bool) -> np.ndarray:
    bits = np.ascontiguousarray(bits).view(np.uint16)
    if bf16:
        return (bits.astype(np.uint32) << 16).view(np.float32)
    return bits.view(np.float16).astype(np.float32)


def ulp_of(ref_f32: np.ndarray, bf16: bool) -> np.ndarray:
    """Spacing of the output type at |ref| (fp16: 10 explicit mantissa bits, bf16: 7)."""
    mant = 7 if bf16 else 10
    min_exp = -126 if bf16 else -14
    a = np.abs(ref_f32).astype(np.float64)
    e = np.floor(np.log2(np.maximum(a, 2.0 ** min_exp)))
    return 2.0 ** (e - mant)


def out_tensor_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().view(torch.int16).cpu().numpy().view(np.uint16)


class OutStats(float):
    """Fraction of bit-identical outputs (the float value), plus `via_reorder`: how many elements
    met the criterion only through the re-association bound, and `size`."""
    via_reorder = 0
    size = 0


# Running totals over a test session: all comparisons, and per workload configuration ("c1" .. "c5"; everything
# else under "other").  conftest.py prints them in the terminal summary; tests/test_zy_tolerance_accounting.py
# asserts the configurations' share.
VIA_REORDER_TOTAL = {"elements": 0, "via_reorder": 0, "worst_x_strict": 0.0}
VIA_REORDER_BY_CONFIG = {}

# Elements of one comparison that may pass only through the re-association bound: parts per million of its size
# (and never fewer than two elements: a 16 x 1024 output is 61 ppm an element).  What randomised sweeps of the
# kernels have shown so far: one or two such elements in a problem of 16 000 .. 676 000 outputs, most problems none.
MAX_VIA_REORDER_PPM = 100.0


def assert_out_close(gpu_bits, ref_bits, bf16, reorder_bound=None, what="", max_via_reorder_ppm=MAX_VIA_REORDER_PPM,
                     config=None):
    """The output criterion of the path: every element within 1 ULP of the output type OR within
    rtol 1e-3 of the oracle.  `reorder_bound` (optional, per element) additionally admits the fp32
    rounding noise of summing the per-group terms in another order (split-K, k-parts, the zero-point
    term through fp32 MFMAs), which is what limits elements whose terms cancel to almost zero; pass
    None where the kernel sums in the oracle's order.  The elements that needed that third term are
    counted (`.via_reorder` of the result, the session totals above) and their share is asserted:
    at most `max_via_reorder_ppm` of the comparison's elements (two elements at least)."""
    g, r = bits_to_f32(gpu_bits, bf16), bits_to_f32(ref_bits, bf16)
    assert np.isfinite(g).all(), f"{what}: non-finite GPU output"
    diff = np.abs(g.astype(np.float64) - r.astype(np.float64))
    strict = np.maximum(ulp_of(r, bf16), 1e-3 * np.abs(r))
    tol = strict if reorder_bound is None else np.maximum(strict, reorder_bound)
    bad = diff > tol
    assert not bad.any(), (f"{what}: {int(bad.sum())} of {bad.size} outputs off; worst |diff|/tol = "
                           f"{float((diff / tol).max()):.3g} at {np.unravel_index(np.argmax(diff / tol), diff.shape)}")
    stats = OutStats((np.ascontiguousarray(gpu_bits).view(np.uint16) == np.ascontiguousarray(ref_bits).view(np.uint16)).mean())
    stats.via_reorder = int((diff > strict).sum())
    stats.size = int(diff.size)
    worst = float((diff / strict).max()) if diff.size else 0.0
    if config is None:
        config = what[:2] if what[:2] in ("c1", "c2", "c3", "c4", "c5") and what[2:3] in ("_", " ", "") else "other"
    for tot in (VIA_REORDER_TOTAL, VIA_REORDER_BY_CONFIG.setdefault(config, {"elements": 0, "via_reorder": 0, "worst_x_strict": 0.0})):
        tot["elements"] += stats.size
        tot["via_reorder"] += stats.via_reorder
        tot["worst_x_strict"] = max(tot["worst_x_strict"], worst if stats.via_reorder else 0.0)
    if stats.via_reorder:
        print(f"{what}: {stats.via_reorder} of {stats.size} outputs beyond rtol 1e-3 / 1 ULP, inside the re-association bound "
              f"(worst {worst:.3g} x the strict tolerance)", flush=True)
    allowed = max(2, int(max_via_reorder_ppm * 1e-6 * stats.size))
    assert stats.via_reorder <= allowed, (f"{what}: {stats.via_reorder} of {stats.size} outputs pass only through the "
                                          f"re-association bound (at most {allowed} allowed)")
    return stats


def via_reorder_summary():
    """One line per configuration seen so far, then the total."""
    lines = []
    for name in sorted(VIA_REORDER_BY_CONFIG):
        t = VIA_REORDER_BY_CONFIG[name]
        lines.append(f"{name}: {t['via_reorder']} of {t['elements']} outputs beyond rtol 1e-3 / 1 ULP "
                     f"(inside the re-association bound; worst {t['worst_x_strict']:.3g} x strict)")
    t = VIA_REORDER_TOTAL
    lines.append(f"all comparisons: {t['via_reorder']} of {t['elements']} outputs beyond rtol 1e-3 / 1 ULP "
                 f"({1e6 * t['via_reorder'] / max(t['elements'], 1):.3g} ppm; worst {t['worst_x_strict']:.3g} x strict)")
    return lines


def reorder_bound(acc: np.ndarray, scale_half: np.ndarray, s_a: np.ndarray) -> np.ndarray:
    """G * 2^-24 * s_a[m] * sum_g |acc[m,n,g]| * scale[g,n]: worst-case drift of an fp32 sum of the
    per-group terms under re-association."""
    s = np.asarray(scale_half, np.float16).astype(np.float64)
    mag = np.einsum("mng,gn->mn", np.abs(acc).astype(np.float64), s)
    return acc.shape[2] * 2.0 ** -24 * mag * np.asarray(s_a, np.float64)[:, None]


@functools.lru_cache(maxsize=8)
def _quantized_weight(n, k, g, mode, dist, seed):
    return workloads.make_quantized_weight(workloads.Case("w", 1, n, k, group_size=g, mode=mode, weight_dist=dist, seed=seed))


def quantized_weight(case):
    """make_quantized_weight, memoised on everything the weight depends on (M does not matter)."""
    return _quantized_weight(case.N, case.K, case.group_size, case.mode, case.weight_dist, case.seed)


def device_inputs(ops, case, packed, scales, zero, x_half):
    """Upload one case: returns (W2A8Weight, x tensor)."""
    uniform = case.zp_const
    w = ops.repack_w2(packed, scales, None if uniform is not None else zero, case.group_size,
                      zp_const=uniform if uniform is not None else 0)
    x = torch.from_numpy(x_half).cuda()
    return w, x


def torch_dtype(case):
    return torch.bfloat16 if case.out_dtype == "bfloat16" else torch.float16


def small_case(M, N, K, g, mode, seed, out_dtype="float16", outliers=False):
    return workloads.Case("t", M, N, K, group_size=g, mode=mode, out_dtype=out_dtype,
                          weight_dist="uniform" if mode == "asym" else "normal", outliers=outliers, seed=seed)
