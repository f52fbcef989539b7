"""bench.py without a GPU: every workload the usage line names exists, every committed rocprofv3 summary that bench.py
reads its `traffic` figures from is there and parses, and a multi-GPU request is refused with a message."""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_usage_line_names_every_workload():
    usage = re.search(r"--workload ([\w|]+)\]", bench.__doc__).group(1).split("|")
    assert sorted(usage) == sorted(bench.WORKLOADS)


def test_profiles_behind_the_traffic_figures_exist_and_parse():
    for key, (fname, kernels, algorithmic) in bench.PROFILE_OF.items():
        assert key in bench.WORKLOADS, key
        path = os.path.join(ROOT, "profiles", fname)
        assert os.path.exists(path), path
        text = open(path).read()
        assert f"--workload {key} " in text, (fname, "was not made by the workload it is filed under")
        t = bench.traffic_from_profile(key)
        assert t is not None, fname
        assert t["source"] == "profiles/" + fname and t["algorithmic_bytes"] == algorithmic
        # the counters see at least the compulsory traffic (reads can hit in cache: a loose lower bound) and no more
        # than an order of magnitude above it
        total = t["fetch_bytes"] + t["write_bytes"]
        assert 0.4 * algorithmic <= total <= 20 * algorithmic, (key, total, algorithmic)
        for k in kernels:
            assert k in text, (fname, k)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr) or "1 GPU" in (r.stdout + r.stderr) or "single" in (r.stdout + r.stderr).lower()
