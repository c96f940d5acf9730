"""Collected after the parity tests (and before the last file): the output-tolerance accounting of the session.

Every comparison of a GPU output with the oracle goes through parity_utils.assert_out_close, which holds each
element to 1 ULP of the output type or rtol 1e-3 and, where a kernel sums the per-group terms in another order than
the oracle, additionally admits the fp32 re-association bound.  The elements that needed that third term are counted
per workload configuration; here the counts of the five configurations are printed and their share is asserted.
Run alone, nothing has been counted and the test only says so.
"""
import pytest

import parity_utils as pu

pytestmark = pytest.mark.gpu

MAX_PPM = 20.0   # of all compared outputs of one configuration


def test_share_of_outputs_that_pass_only_through_the_reorder_bound(gpu_ops):
    for line in pu.via_reorder_summary():
        print(line, flush=True)
    if not pu.VIA_REORDER_TOTAL["elements"]:
        pytest.skip("no output comparison has run in this session")
    for name in ("c1", "c2", "c3", "c4", "c5"):
        t = pu.VIA_REORDER_BY_CONFIG.get(name)
        if t is None:
            continue
        allowed = max(2, int(MAX_PPM * 1e-6 * t["elements"]))
        assert t["via_reorder"] <= allowed, f"{name}: {t['via_reorder']} of {t['elements']} outputs beyond rtol 1e-3 / 1 ULP"
