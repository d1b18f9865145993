"""bench.py's command-line contract that needs no GPU: more than one GPU is refused with a message, and a machine
without a GPU gets a plain error instead of a fallback."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused():
    r = run("--gpus", "2")
    assert r.returncode == 2 and "ONE GPU" in r.stderr and r.stdout == ""


def test_unknown_workload_is_an_argument_error():
    r = run("--workload", "nope")
    assert r.returncode == 2 and "invalid choice" in r.stderr
