"""bench.py's command line (no GPU needed): one GPU only, and a loud failure where no device is present."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args, env=None):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300,
                          env={**os.environ, **(env or {})})


def test_more_than_one_gpu_is_refused_with_a_message():
    for r in (run("--gpus", "2"), run(env={"WORLD_SIZE": "2"})):
        assert r.returncode != 0 and "--gpus 1" in r.stderr and r.stdout.strip() == ""


def test_no_device_fails_loudly():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    r = run("--steps", "2", "--warmup", "1", "--skip-cpu")
    assert r.returncode != 0 and "unavailable" in r.stderr and r.stdout.strip() == ""
