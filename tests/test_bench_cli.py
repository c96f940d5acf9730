"""The benchmark's command line and constants, without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert "exactly one GPU" in r.stderr and "--gpus 2" in r.stderr
    assert r.stdout.strip() == ""          # no JSON line for a run that measured nothing


def test_constants_against_the_workload():
    sys.path.insert(0, ROOT)
    import bench
    from slimkernels_amd import workloads
    assert bench.HBM_PEAK_GBPS == 8000.0 and bench.INT8_PEAK_TOPS == 5000.0
    step_bytes = sum(workloads.algorithmic_bytes(c) for c in workloads.config_cases("c2"))
    assert len(workloads.config_cases("c2")) == 24
    # counter-measured HBM traffic of one launch: at least the algorithmic bytes, and not much more
    assert 1.0 <= bench.MEASURED_TRAFFIC_BYTES_PER_LAUNCH / step_bytes < 1.15
