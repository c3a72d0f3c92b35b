"""bench.py's command line on a machine without a GPU: one GPU only, and a clear refusal otherwise."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*flags):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], capture_output=True, text=True,
                          cwd=ROOT, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_help_lists_the_other_workloads():
    r = _run("--help")
    assert r.returncode == 0
    for flag in ("--layers", "--e2e", "--sweep", "--rel", "--window", "--no-cpu", "--preheat-ms"):
        assert flag in r.stdout
