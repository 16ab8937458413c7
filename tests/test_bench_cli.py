"""bench.py contract checks that need no GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert p.returncode == 2
    assert "one GPU only" in p.stderr and p.stdout.strip() == ""


def test_bench_sources_name_the_baseline_metric_and_workloads():
    src = open(os.path.join(ROOT, "bench.py")).read()
    for key in ('"metric"', '"roofline"', '"cpu_baseline"', '"vs_baseline"', '"config"', '"workload"', '"traffic"'):
        assert key in src
    for w in ("c1", "c2", "c3", "c4", "c5"):
        assert f'"{w}"' in src
