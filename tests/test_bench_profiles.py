"""bench.py takes its HBM-traffic figures from the tracked rocprofv3 summaries:
the parser must find the file of every profiled workload and read the dominant
kernel's FETCH_SIZE / WRITE_SIZE lines from it (no GPU needed)."""
import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_headline_traffic_is_what_the_profile_says():
    traffic, source, trace = bench.measured_traffic("min_bmm_large")
    assert source == "profiles/min_kernel_min_bmm_large.txt"
    text = open(os.path.join(ROOT, source)).read()
    fetch = float(re.search(r"cmk::min_kernel<[^\n]*FETCH_SIZE\s+n=\d+ avg=(\S+)", text).group(1))
    write = float(re.search(r"cmk::min_kernel<[^\n]*WRITE_SIZE\s+n=\d+ avg=(\S+)", text).group(1))
    assert traffic == (2 * fetch + write) * 1024
    assert any("min_kernel" in k for k in trace) and any("min_fold_kernel" in k for k in trace)


def test_every_kernel_summary_is_found_by_its_workload_name():
    names = []
    for f in sorted(os.listdir(os.path.join(ROOT, "profiles"))):
        m = re.match(r"([a-z_]+_kernel)_(.+)\.txt$", f)
        if not m or m.group(2).startswith("floor"):
            continue
        names.append(m.group(2))
        traffic, source, _ = bench.measured_traffic(m.group(2))
        assert source == "profiles/" + f, (f, source)
        assert traffic and traffic > 0, f
    assert "topk_bmm" in names and "bmm" in names and "mbmm" in names


def test_unknown_workload_has_no_traffic():
    assert bench.measured_traffic("no_such_workload") == (None, None, {})
