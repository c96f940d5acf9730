"""The benchmark / parity workloads of the W2A8 path and their seeded synthetic inputs.

Five configurations (names c1..c5):
  c1  M=16, N=K=4096, group 128, symmetric levels, fp16 out (the CPU-runnable case)
  c2  decode sweep, M in {1,2,4,8,16,32} over Llama-3-8B linears, 0.1 % outlier channels
  c3  prefill, M in {512,2048,4096}, N x K in {14336x4096, 4096x14336}
  c4  70B-class FFN shapes, group 64, bf16 out, M in {1,16,128,2048}
  c5  asymmetric codes with per-group zero-points, ragged shapes
Weights are float16 draws quantised by slimkernels_amd.quantization (host numpy);
activations are float16 draws.  Generator seeds: weight = seed, activation = seed + 1.
"""
import dataclasses

import numpy as np
import torch

from .quantization import prepare_w2


def _to_half(x32: np.ndarray) -> np.ndarray:
    """float32 -> float16, round-to-nearest-even (torch's CPU cast: same values as numpy's, much faster)."""
    return torch.from_numpy(np.ascontiguousarray(x32, np.float32)).to(torch.float16).numpy()


def _to_float(x16: np.ndarray) -> np.ndarray:
    return torch.from_numpy(np.ascontiguousarray(x16)).to(torch.float32).numpy()


@dataclasses.dataclass(frozen=True)
class Case:
    config: str
    M: int
    N: int
    K: int
    group_size: int = 128
    mode: str = "sym"            # "sym" | "asym" | "ref"
    out_dtype: str = "float16"   # "float16" | "bfloat16"
    weight_dist: str = "normal"  # "normal": N(0, 0.02) | "uniform": U[-0.05, 0.05]
    outliers: bool = False       # scale ceil(0.001 K) activation channels by 20
    seed: int = 0

    @property
    def name(self):
        return f"{self.config}_M{self.M}_N{self.N}_K{self.K}_g{self.group_size}_{self.mode}"

    @property
    def zp_const(self):
        return {"sym": 2, "ref": 1}.get(self.mode)


LLAMA8B_LINEARS = {"qo": (4096, 4096), "kv": (1024, 4096), "gate_up": (14336, 4096), "down": (4096, 14336)}
DECODE_M = (1, 2, 4, 8, 16, 32)


def config_cases(config: str):
    if config == "c1":
        return [Case("c1", 16, 4096, 4096)]
    if config == "c2":
        return [Case("c2", m, n, k, outliers=True) for (n, k) in LLAMA8B_LINEARS.values() for m in DECODE_M]
    if config == "c3":
        return [Case("c3", m, n, k) for (n, k) in ((14336, 4096), (4096, 14336)) for m in (512, 2048, 4096)]
    if config == "c4":
        return [Case("c4", m, n, k, group_size=64, out_dtype="bfloat16")
                for (n, k) in ((28672, 8192), (8192, 28672)) for m in (1, 16, 128, 2048)]
    if config == "c5":
        return [Case("c5", 77, 11008, 4096, mode="asym", weight_dist="uniform"),
                Case("c5", 1, 5120, 13824, mode="asym", weight_dist="uniform")]
    raise ValueError(config)


def make_weight(case: Case) -> np.ndarray:
    """float16 [N, K] weight draw (chunked so the float64 generator output stays small)."""
    rng = np.random.default_rng(case.seed)
    w = np.empty((case.N, case.K), np.float16)
    rows = max(1, (1 << 24) // case.K)
    for r0 in range(0, case.N, rows):
        r1 = min(case.N, r0 + rows)
        if case.weight_dist == "normal":
            w[r0:r1] = _to_half(rng.standard_normal((r1 - r0, case.K), dtype=np.float32) * np.float32(0.02))
        else:
            w[r0:r1] = _to_half(rng.uniform(-0.05, 0.05, (r1 - r0, case.K)).astype(np.float32))
    return w


def make_activation(case: Case) -> np.ndarray:
    """float16 [M, K] activation draw, N(0,1), optionally with x20 outlier channels."""
    rng = np.random.default_rng(case.seed + 1)
    x = rng.standard_normal((case.M, case.K), dtype=np.float32)
    if case.outliers:
        n_out = int(np.ceil(0.001 * case.K))
        cols = rng.choice(case.K, size=n_out, replace=False)
        x[:, cols] *= np.float32(20.0)
    return _to_half(x)


def make_quantized_weight(case: Case):
    """(packed uint8 [N, K/4], scales float16 [G, N], zero-points uint8 [G, N])."""
    w = make_weight(case)
    N = case.N
    packed = np.empty((N, case.K // 4), np.uint8)
    G = case.K // case.group_size
    scales = np.empty((G, N), np.float16)
    zero = np.empty((G, N), np.uint8)
    rows = max(64, (1 << 25) // case.K)
    for r0 in range(0, N, rows):  # quantise a slab of channels at a time (bounded temporaries)
        r1 = min(N, r0 + rows)
        p, s, z = prepare_w2(_to_float(w[r0:r1]), case.group_size, case.mode)
        packed[r0:r1], scales[:, r0:r1], zero[:, r0:r1] = p, s, z
    return packed, scales, zero


def algorithmic_bytes(case: Case) -> int:
    """Compulsory HBM traffic of one GEMM call: packed codes + fp16 scales (+ 2-bit zero-points)
    + int8 activations + token scales + per-group row sums + the output, each counted once."""
    M, N, K, G = case.M, case.N, case.K, case.K // case.group_size
    b = N * K // 4 + 2 * N * G + M * K + 4 * M + 4 * M * G + 2 * M * N
    if case.mode == "asym":
        b += N * G // 4
    return b


def algorithmic_ops(case: Case) -> int:
    return 2 * case.M * case.N * case.K
