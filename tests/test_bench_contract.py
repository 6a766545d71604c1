"""bench.py's command line contract that needs no GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert p.returncode == 2
    assert "ONE GPU" in p.stderr and p.stdout.strip() == ""


def test_workloads_are_listed():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0
    for w in ("painn_layer", "neighbour", "products", "denoiser", "stress", "polymer"):
        assert w in p.stdout
