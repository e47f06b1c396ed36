"""bench.py's command line, as far as it can be checked without a GPU: one GPU only, and a traffic figure is never
quoted without the profile it was read from."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       cwd=ROOT, timeout=120)
    assert r.returncode == 2
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_traffic_figures_name_their_profile():
    sys.path.insert(0, ROOT)
    import bench
    assert bench.MEASURED_TRAFFIC, "counter figures for the headline kernels"
    assert os.path.isfile(os.path.join(ROOT, bench.TRAFFIC_SOURCE))
    text = open(os.path.join(ROOT, bench.TRAFFIC_SOURCE)).read().replace(" ", "")
    for key, (read, written) in bench.TRAFFIC_READ_WRITTEN.items():
        assert str(read) in text, (key, read)          # the profile's "x2 = bytes read" column
        assert bench.MEASURED_TRAFFIC[key] == read + written
