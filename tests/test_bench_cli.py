"""The benchmark's command line where no GPU is needed: it measures one GPU only and says so."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args, env=None):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True, timeout=300, env=env)


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = run_bench("--gpus", "2")
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr and proc.stdout.strip() == ""


def test_a_multi_rank_launch_is_refused_too():
    proc = run_bench("--gpus", "1", env=dict(os.environ, WORLD_SIZE="2", RANK="0", LOCAL_RANK="0"))
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr and proc.stdout.strip() == ""
