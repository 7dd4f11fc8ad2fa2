"""The parts of bench.py's contract that can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr


def test_side_workloads_are_listed():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0
    for name in ("linear_11008", "conv2d_256", "mlp_3072_8192", "fwd_dynamic_4096"):
        assert name in proc.stdout
