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


def test_traffic_records_name_kernels_the_library_still_carries():
    """profiles/traffic.json ties each measured HBM traffic figure to the kernel it was measured on. A record whose
    kernel is no longer in the built library is stale (the kernel was replaced or renamed): measure again, or drop it."""
    import json
    from skainet_amd import _lib
    with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
        rec = json.load(f)
    assert rec["calibration"]["FETCH_SIZE_factor"] > 1.5 and rec["calibration"]["WRITE_SIZE_factor"] > 0.5
    blob = open(_lib.HIP_LIB_PATH, "rb").read()
    import bench
    known = set(bench.WORKLOADS) | set(bench.ATTENTION_WORKLOADS) | set(bench.DECODER_WORKLOADS)
    for name, r in rec["workloads"].items():
        assert name in known, name
        assert r["bytes_per_launch"] > 0
        assert r["kernel"].encode() in blob, f"{name}: kernel {r['kernel']} is not in the library any more"
        assert os.path.exists(os.path.join(ROOT, r["summary"])), r["summary"]
    # the record of the default workload belongs to the kernel the dispatch takes for it (named in the launcher's source)
    head = rec["workloads"].get("q4k_gemv_11008x4096_b1")
    if head is not None:
        src = open(os.path.join(ROOT, "skainet_amd", "csrc", "gemv_q4k_mfma.hip")).read()
        assert f'note_kernel("{head["kernel"]}")' in src
