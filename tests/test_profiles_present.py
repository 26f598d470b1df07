"""No GPU: the rocprofv3 summaries the bench line's roofline objects rest on exist and say something."""
import glob
import json
import os

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROFILES = os.path.join(ROOT, "profiles")


def test_no_summary_is_empty():
    files = glob.glob(os.path.join(PROFILES, "*.md")) + glob.glob(os.path.join(PROFILES, "*.txt"))
    assert files
    for f in files:
        text = open(f).read()
        assert len(text) > 400 and "rocprofv3" in text, f  # the command that made it is in the file


def test_every_priced_kernel_has_its_summary_and_traffic_figure():
    traffic = json.load(open(os.path.join(PROFILES, "traffic.json")))
    for key, (kernel, workload) in bench.ROOFLINE_KERNELS.items():
        path = os.path.join(PROFILES, bench.profile_file(kernel, workload))
        assert os.path.exists(path), (key, path)
        text = open(path).read()
        assert kernel in text and "avg=" in text, path           # per-kernel durations
        assert "FETCH_SIZE" in text and "WRITE_SIZE" in text, path  # and the HBM counters
        assert workload in traffic.get(kernel, {}), (kernel, workload)
        assert bench.load_traffic(kernel, workload) > 0
