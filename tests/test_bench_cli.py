"""bench.py's command line, as far as it can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    # the build is single-GPU: no collectives, no sharding; the bench says so instead of running one rank's share
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 2
    assert "one GPU only" in r.stderr and r.stdout == ""


def test_workloads_are_listed_in_the_help():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0
    for name in ("default", "decode", "prefill", "mixtral_decode", "mixtral_prefill", "qwen3_235b_prefill"):
        assert name in r.stdout
