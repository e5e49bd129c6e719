"""The benchmark's command line, as far as it can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], cwd=ROOT, capture_output=True,
                          text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode == 2
    assert "one GPU only" in r.stderr
    assert r.stdout.strip() == ""


def test_help_lists_the_measurement_switches():
    r = _run("--help")
    assert r.returncode == 0
    for flag in ("--steps", "--warmup", "--all", "--only", "--no-cpu", "--kernels-only"):
        assert flag in r.stdout
