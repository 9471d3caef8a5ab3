"""bench.py command-line contract that can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_without_a_gpu_it_fails_loudly_instead_of_falling_back():
    import torch
    if torch.cuda.is_available():
        return
    r = _run("--steps", "1", "--warmup", "0")
    assert r.returncode != 0
    assert "no GPU" in r.stderr and r.stdout.strip() == ""
