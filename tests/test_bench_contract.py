"""The command-line contract of bench.py that can be checked without a GPU: one GPU only, and a product path
that refuses to run without one instead of falling back to the CPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=300, cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "--gpus must be 1" in r.stderr + r.stdout
    assert not r.stdout.strip().startswith("{")          # no result line


def test_no_result_line_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        import pytest
        pytest.skip("this box has a GPU")
    r = _run("--steps", "1", "--warmup", "0", "--cpu-seconds", "0")
    assert r.returncode != 0 and not r.stdout.strip().startswith("{")
