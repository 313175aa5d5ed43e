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


def test_the_checker_is_imported_only_by_the_parity_and_cpu_baseline_legs():
    """`oracle` may only be imported under `if parity:` or `if cpu:` inside a workload (never at module level,
    never on the timed path), so `--no-cpu --no-parity` runs without the checker."""
    import ast
    tree = ast.parse(open(os.path.join(ROOT, "bench.py")).read())
    guarded, all_imports = set(), set()

    def is_oracle(node):
        if isinstance(node, ast.Import):
            return any(a.name.split(".")[0] == "oracle" for a in node.names)
        return isinstance(node, ast.ImportFrom) and (node.module or "").split(".")[0] == "oracle"

    for node in ast.walk(tree):
        if is_oracle(node):
            all_imports.add(node.lineno)
        if isinstance(node, ast.If) and isinstance(node.test, ast.Name) and node.test.id in ("cpu", "parity"):
            for sub in ast.walk(node):
                if is_oracle(sub):
                    guarded.add(sub.lineno)
    assert all_imports and all_imports == guarded, sorted(all_imports - guarded)
