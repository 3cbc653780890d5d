"""Host-side pieces of bench.py that need no GPU: the one-GPU rule, the mode a configuration is timed
in, and the traffic figure read back from the committed hardware-counter summaries."""
import os
import subprocess
import sys
import types

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_more_than_one_gpu_is_refused():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert out.returncode == 2
    assert "ONE GPU" in out.stderr and out.stdout.strip() == ""


def test_accumulate_mode_per_configuration():
    a = types.SimpleNamespace(accumulate="auto")
    assert [bench.accumulate_mode(a, c) for c in (1, 2, 3, 4, 5)] == ["exact", "exact", "exact", "exact", "fast"]
    assert bench.accumulate_mode(types.SimpleNamespace(accumulate="fast"), 3) == "fast"
    assert bench.accumulate_mode(types.SimpleNamespace(accumulate="exact"), 5) == "exact"


def test_traffic_comes_from_the_committed_profiles():
    # config 3 moves about what it needs (636 MB of rows + 48 MB of indices and weights in, 43.5 MB out);
    # config 5 fetches less than its 13 GB of row bytes (hot rows come out of the caches) and writes 3.4 GB;
    # config 4 moves several times its 64 MB of row bytes (36-byte rows out of 128-byte lines)
    t3, t4, t5 = (bench.traffic_from_profile(c) for c in (3, 4, 5))
    assert 600e6 < t3 < 800e6
    assert 300e6 < t4 < 700e6
    assert 7e9 < t5 < 14e9
    assert bench.traffic_from_profile(1) is None  # no summary committed for the single-table configurations
