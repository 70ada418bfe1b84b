"""bench.py's command line as the driver uses it: more than one GPU is refused with a message
(every box has one GPU), and on a machine without a GPU the default run stops with a clear error
instead of measuring anything on the CPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=300, cwd=ROOT)


def test_more_than_one_gpu_is_refused():
    r = run("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert r.returncode != 0
    assert "one GPU" in r.stderr or "--gpus 1" in r.stderr, r.stderr
    assert r.stdout.strip() == ""


def test_no_gpu_no_numbers():
    import torch
    if torch.cuda.is_available():
        import pytest
        pytest.skip("this machine has a GPU")
    r = run("--steps", "1", "--warmup", "0", "--no-cpu-baseline")
    assert r.returncode != 0
    assert r.stdout.strip() == ""           # no JSON line without a measurement
