"""CPU checks of the measurement contract: what bench.py refuses, and that the committed profile
summaries cover every bench workload."""
import json
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _workloads():
    src = open(os.path.join(ROOT, "bench.py")).read()
    m = re.search(r'choices=\[([^\]]+)\]', src)
    return [w.strip().strip('"') for w in m.group(1).split(",")]


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)
    assert not r.stdout.strip().startswith("{")              # no result line for a configuration that was not run


# Workloads added after the last profiling session.  When a profile lands the name must leave this
# list (the test below insists), so the list cannot go stale.
NOT_YET_PROFILED = {"decode_fp8_h128"}


def test_profiles_cover_the_bench_workloads():
    traffic = json.load(open(os.path.join(ROOT, "profiles", "hbm_traffic.json")))
    names = os.listdir(os.path.join(ROOT, "profiles"))
    for wl in _workloads():
        if wl in NOT_YET_PROFILED:
            assert wl not in traffic and not [n for n in names if n.endswith(f"_{wl}.md")], f"{wl} is profiled: take it off the list"
            continue
        assert wl in traffic, f"no HBM traffic figure for {wl}"
        assert traffic[wl]["hbm_bytes_per_launch"] > 0 and traffic[wl]["algorithmic_bytes_per_launch"] > 0
        summary = [n for n in names if n.endswith(f"_{wl}.md")]
        assert summary, f"no rocprofv3 summary for {wl}"
        text = open(os.path.join(ROOT, "profiles", summary[0])).read()
        assert "rocprofv3 --kernel-trace --stats" in text and f"--workload {wl}" in text
        assert traffic[wl]["kernel"] in summary[0]
