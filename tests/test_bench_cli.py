"""bench.py's command line, as far as it can be checked without a GPU: more than one GPU is
refused with a message that says why, and without a device the script stops before measuring
anything (no CPU fallback is ever timed)."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args],
                          capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "ONE MI355X" in r.stderr and "--gpus must be 1" in r.stderr
    assert r.stdout.strip() == ""


def test_without_a_gpu_nothing_is_measured():
    import torch
    if torch.cuda.is_available():
        import pytest
        pytest.skip("a GPU is present")
    r = _run("--steps", "1", "--warmup", "0")
    assert r.returncode != 0
    assert "needs a GPU" in r.stderr
    assert r.stdout.strip() == ""
