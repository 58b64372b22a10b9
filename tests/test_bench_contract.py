"""bench.py contract that needs no GPU: more than one GPU is refused with a message, and the algorithmic byte count of the
headline workload is the documented 204.05 MB."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_headline_algorithmic_bytes():
    sys.path.insert(0, ROOT)
    import bench
    n = bench.scan_algorithmic_bytes(8, 2048, 1536, 16, 2, gated=True)
    assert abs(n - 204.05e6) < 0.01e6
    assert bench.scan_algorithmic_bytes(8, 2048, 1536, 16, 2, gated=False) < n
