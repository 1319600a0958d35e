"""bench.py's command line: what it refuses without touching a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], cwd=ROOT,
                          capture_output=True, text=True, timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = run("--gpus", "2")
    assert r.returncode != 0
    assert "single GPU" in (r.stdout + r.stderr)
    assert "{" not in r.stdout  # no result line


def test_unknown_workload_is_refused():
    r = run("--workload", "nonsense")
    assert r.returncode != 0
