"""The parts of bench.py's contract that can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          cwd=ROOT, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = run("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_workload_names_and_data_choices_are_validated():
    assert run("--workload", "no_such_workload").returncode != 0
    assert run("--data", "ones").returncode != 0
