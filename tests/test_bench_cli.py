"""bench.py's command line where no GPU is needed: it measures one GPU and says so when asked for more."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120, cwd=ROOT)
    assert p.returncode != 0 and "one GPU" in p.stderr and p.stdout.strip() == ""


def test_bench_refuses_out_of_range_options():
    for flags in (["--comms", "5"], ["--depth", "17"], ["--pools", "0"]):
        p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + flags, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120, cwd=ROOT)
        assert p.returncode != 0 and "must be" in p.stderr
