import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (oracle/w2a8_oracle.py + its C library, built on first use)."""
    from oracle import w2a8_oracle
    w2a8_oracle.lib()
    return w2a8_oracle


@pytest.fixture(scope="session")
def gpu_ops():
    """The product's GPU entry points; skips when no GPU is visible."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from slimkernels_amd import torch as ops  # raises if the HIP library is missing
    return ops


def pytest_terminal_summary(terminalreporter):
    """Output-tolerance accounting of the GPU parity tests: how many compared outputs lay beyond rtol 1e-3 / 1 ULP and
    passed through the re-association bound only (per workload configuration, then in total)."""
    try:
        import parity_utils as pu
    except ImportError:
        return
    if pu.VIA_REORDER_TOTAL["elements"]:
        terminalreporter.write_line("output tolerance accounting (GPU outputs against the oracle):")
        for line in pu.via_reorder_summary():
            terminalreporter.write_line("  " + line)
