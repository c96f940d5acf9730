#!/usr/bin/env python3
"""Writes tests/golden/w2a8_small.npz: small seeded W2A8 cases with every intermediate result.

The vectors are build-authored (the upstream repository has no fixture for the int8 / int32 /
epilogue part of the path; its own known-answer vectors for pack and quantize are kept verbatim
in tests/test_reference_contract.py).  They were produced by the CPU oracle once it had passed
tests/test_oracle.py, and are frozen here so that a later change to the oracle or the kernels
that alters any bit shows up as a diff against committed data.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import w2a8_oracle as orc  # noqa: E402
from slimkernels_amd import workloads  # noqa: E402

CASES = [
    # name, M, N, K, group, mode, out dtype
    ("sym_g128", 4, 8, 256, 128, "sym", "float16"),
    ("sym_g64_bf16", 3, 8, 256, 64, "sym", "bfloat16"),
    ("asym_g128", 4, 8, 256, 128, "asym", "float16"),
    ("ref_g64", 2, 8, 128, 64, "ref", "float16"),
]


def main():
    out = {}
    for name, M, N, K, g, mode, odt in CASES:
        case = workloads.Case("golden", M, N, K, group_size=g, mode=mode, out_dtype=odt,
                              weight_dist="uniform" if mode == "asym" else "normal", seed=100 + len(out))
        packed, scales, zero = workloads.make_quantized_weight(case)
        x = workloads.make_activation(case)
        ref = orc.reference_forward(x, packed, scales, zero, g, out_bf16=(odt == "bfloat16"))
        for key, val in dict(x=x.view(np.uint16), packed=packed, scales=scales.view(np.uint16), zp=zero,
                             q=ref["q"], s_a=ref["s_a"], rowsum=ref["rowsum"], acc=ref["acc"],
                             out_bits=ref["out_bits"]).items():
            out[f"{name}/{key}"] = val
        out[f"{name}/meta"] = np.array([M, N, K, g, {"ref": 0, "sym": 1, "asym": 2}[mode], int(odt == "bfloat16")])
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "w2a8_small.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
