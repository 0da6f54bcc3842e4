"""bench.py contract checks that need no GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode != 0
    assert "ONE GPU" in proc.stderr and proc.stdout.strip() == ""


def test_workloads_cover_the_reference_gpu_configurations():
    sys.path.insert(0, ROOT)
    import bench
    assert bench.WORKLOADS["headline"][1:6] == (256, 64, 1024, 2, 3)
    assert bench.WORKLOADS["config2"][1:6] == (128, 32, 512, 2, 3)
    assert bench.WORKLOADS["config4"][1:6] == (512, 16, 2048, 1, 3)
    assert bench.WORKLOADS["config5"][1:7] == (4096, 256, 256, 2, 3, True)
    assert bench.HBM_PEAK_GBS == 8000.0
