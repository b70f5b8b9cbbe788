"""The parts of ``bench.py`` that need no GPU: it measures one GPU only, and its workload table
matches the configurations it documents."""

import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 2
    assert "one GPU" in proc.stderr and "--gpus must be 1" in proc.stderr
    assert proc.stdout.strip() == ""  # no JSON line is printed for a refused run


def test_workload_table():
    sys.path.insert(0, str(ROOT))
    import bench

    assert bench.WORKLOADS["c1"] == ("ag", 4096, 4096, 1024, 128, "f16")
    assert bench.WORKLOADS["c2"][:4] == ("ag", 8192, 4096, 1024)
    assert bench.WORKLOADS["c3"] == ("rs", 8192, 4096, 2048, 128, "f16")
    assert bench.WORKLOADS["c4"] == ("rs", 16384, 4096, 2048, 128, "f8")
    assert bench.WORKLOADS["ch1"][0] == "ch"
    assert bench.PEAK_TFLOPS["f16"] == 2500.0 and bench.PEAK_TFLOPS["f8"] == 5000.0 and bench.PEAK_HBM_GBS == 8000.0
    # every measured-traffic constant names a workload and variant that exist
    for (name, variant, macro) in bench.MEASURED_TRAFFIC_BYTES:
        assert name in bench.WORKLOADS and variant in ("s0", "s1", "s2") and macro in (0, 128, 256)
