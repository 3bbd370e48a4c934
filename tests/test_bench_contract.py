"""bench.py's command-line contract, as far as it can be checked without a GPU."""

import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0
    assert "one GPU" in res.stderr


def test_without_a_gpu_it_says_so_instead_of_falling_back():
    import torch

    if torch.cuda.is_available():
        return
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--quick"], capture_output=True, text=True)
    assert res.returncode != 0
    assert "no CPU path" in res.stderr and "{" not in res.stdout


def test_help_names_the_contract_flags():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True)
    for flag in ("--gpus", "--steps", "--warmup"):
        assert flag in res.stdout
