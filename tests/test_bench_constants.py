"""bench.py quotes HBM traffic per launch as constants taken from counter runs; each constant must be the
figure of the committed counter summary it names (the first kernel row of its traffic table)."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_traffic_constants_are_the_figures_of_the_committed_summaries():
    import bench
    assert set(bench.TRAFFIC_SOURCE) == set(bench.MEASURED_TRAFFIC_BYTES)
    for key, path in bench.TRAFFIC_SOURCE.items():
        text = open(os.path.join(ROOT, path)).read()
        section = text[text.index("## HBM traffic per launch"):]
        rows = re.findall(r"^\| `([^`]+)` \| \d+ \| [\d.]+ \| [\d.]+ \| ([\d.]+) \|", section, flags=re.M)
        assert rows, path
        megabytes = float(rows[0][1])   # the dominant kernel comes first
        assert abs(megabytes - bench.MEASURED_TRAFFIC_BYTES[key] / 1e6) <= 0.051, (key, megabytes)
        assert "rocprofv3 --pmc FETCH_SIZE" in section and "rocprofv3 --pmc WRITE_SIZE" in section


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "one GPU" in r.stderr
