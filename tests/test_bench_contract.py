"""bench.py's command-line contract where it can be checked without a GPU: more than one GPU is
refused with a message (the path has no multi-GPU component), and without a HIP device the
benchmark fails loudly instead of measuring anything else."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=300, cwd=ROOT)


def test_more_than_one_gpu_is_refused():
    r = run_bench("--gpus", "2")
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_no_device_no_number():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    r = run_bench("--steps", "1", "--warmup", "0", "--cpu-seconds", "0")
    assert r.returncode == 3
    assert "no CPU fallback" in r.stderr and r.stdout.strip() == ""
