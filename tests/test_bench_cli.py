"""bench.py's command line, as far as it runs without a GPU: more than one GPU is refused with a message, and the
counter traffic quoted in the roofline object is tied to the kernel sources it was measured on."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_counter_traffic_is_quoted_only_for_the_sources_it_was_measured_on(tmp_path, monkeypatch):
    sys.path.insert(0, ROOT)
    import bench
    with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
        t = json.load(f)
    kernel, nbytes = next(iter(t["bytes_per_launch"]["cfg5"].items()))
    if t["kernel_sources_digest"] == bench.kernel_sources_digest():
        assert bench.measured_traffic("cfg5", kernel) == nbytes
    monkeypatch.setattr(bench, "kernel_sources_digest", lambda: "not the digest of any source tree")
    assert bench.measured_traffic("cfg5", kernel) is None
    assert bench.measured_traffic("cfg5", "no such kernel") is None
