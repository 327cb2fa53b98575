"""The command-line contract of bench.py that needs no GPU: more than one GPU is refused with a
message (every measurement here is one rank's share on one GPU), and without a GPU the program
says so instead of measuring anything else."""

import os
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = run("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr) and "--gpus 1" in (r.stdout + r.stderr)
    assert not any(line.startswith("{") for line in r.stdout.splitlines())  # no result line


@pytest.mark.skipif(torch.cuda.is_available(), reason="this box has a GPU")
def test_without_a_gpu_nothing_is_measured():
    r = run("--steps", "1", "--warmup", "0")
    assert r.returncode != 0
    assert "needs a GPU" in (r.stdout + r.stderr)
    assert not any(line.startswith("{") for line in r.stdout.splitlines())
