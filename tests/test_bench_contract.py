"""Host-side contract of bench.py that needs no GPU: the multi-GPU refusal, and the traffic figure it reports comes from
the committed counter summary."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2
    assert "one GPU" in r.stderr
    assert r.stdout.strip() == ""


def test_traffic_figure_comes_from_the_committed_profile():
    sys.path.insert(0, ROOT)
    import bench
    t = bench.committed_traffic("traffic_bytes_per_launch")
    assert t is not None and 1.4e8 < t < 2e9          # above the 147 MB of algorithmic traffic, below absurd
    t = bench.committed_traffic("traffic_bytes_per_launch_masked_forward")
    assert t is not None and 1.3e8 < t < 2e9          # above the 136 MB of algorithmic traffic
    assert bench.committed_traffic("no_such_figure") is None
    text = open(bench.TRAFFIC_PROFILE).read()
    assert "FETCH_SIZE" in text and "WRITE_SIZE" in text and "rocprofv3" in text
