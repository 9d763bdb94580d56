"""Host-side contract of bench.py that needs no GPU: it measures one GPU and says so when asked for
more, its metric is the one BASELINE.json names, and every workload it offers has a profile summary
under profiles/ named for it."""
import json
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)
    assert r.stdout.strip() == ""   # no JSON line that a driver could mistake for a result


def test_metric_is_the_one_baseline_names():
    src = open(os.path.join(ROOT, "bench.py")).read()
    metric = json.load(open(os.path.join(ROOT, "BASELINE.json")))["metric"]
    assert json.dumps(metric)[1:-1] in src or metric in src


def test_every_workload_has_a_profile_summary():
    src = open(os.path.join(ROOT, "bench.py")).read()
    table = re.search(r"WORKLOADS\s*=\s*\{(.*?)\}", src, re.S)
    assert table, "bench.py lists its workloads in a WORKLOADS table"
    names = re.findall(r'"(\w+)"\s*:', table.group(1))
    assert "titans_chunkwise_c3" in names
    have = os.listdir(os.path.join(ROOT, "profiles"))
    for n in names:
        assert any(f.startswith(n) for f in have), f"profiles/ has no summary for {n}"
