"""Builds the two in-tree native libraries of the package.

    libskainet_hip.so    gfx950 kernels + C ABI (hipcc, one object per .hip file under csrc/)
    libskainet_quant.so  host-side GGUF block quantizers (gcc + OpenMP)

hipcc cross-compiles for gfx950 without a GPU. Run as `python -m skainet_amd.build` (add `-v` to echo
the commands, `--jobs N` to compile N files at once).
"""
from __future__ import annotations

import argparse
import concurrent.futures
import os
import shutil
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(PKG, "build")
HIP_SOURCES = ["shim.hip", "dequant.hip", "gemv.hip", "gemv_stream.hip", "gemv_q8_0_mfma.hip", "gemv_q4k.hip", "gemv_q4k_mfma.hip", "gemv_q4k_quads.hip", "gemv_q4k_wide.hip", "gemm.hip", "gemm_q4k_ksw.hip", "gemm_q4k_frag.hip", "rows.hip", "sdpa.hip", "sdpa_decode.hip", "sdpa_prefill.hip", "dense.hip", "elementwise.hip"]
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wno-unused-function",
    # packed FP32 VALU ops are kept out of generated code on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass of hipcc warns that it does not know the GPU-only feature flag: harmless noise
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError(f"command failed ({r.returncode}): {' '.join(cmd)}\n{r.stdout}\n{r.stderr}")
    if err and verbose:
        print(err, file=sys.stderr)


def hipcc() -> str:
    for c in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if c and os.path.exists(c):
            return c
    raise RuntimeError("hipcc not found")


def build_hip(verbose=False, jobs=4, extra_flags=()):
    os.makedirs(OBJ, exist_ok=True)
    cc = hipcc()
    objs = [os.path.join(OBJ, s.replace(".hip", ".o")) for s in HIP_SOURCES]
    cmds = [[cc, *HIP_FLAGS, *extra_flags, "-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(HIP_SOURCES, objs)]
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda c: _run(c, verbose), cmds))
    out = os.path.join(PKG, "libskainet_hip.so")
    _run([cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out + ".tmp", *objs], verbose)
    os.replace(out + ".tmp", out)
    return out


def build_quant(verbose=False):
    out = os.path.join(PKG, "libskainet_quant.so")
    _run(["gcc", "-O2", "-fopenmp", "-fPIC", "-shared", "-fvisibility=hidden", "-o", out + ".tmp",
          os.path.join(CSRC, "ggml_quant.c"), "-lm"], verbose)
    os.replace(out + ".tmp", out)
    return out


def build_all(verbose=False, jobs=4):
    return build_hip(verbose, jobs), build_quant(verbose)


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-v", "--verbose", action="store_true")
    ap.add_argument("--jobs", type=int, default=4)
    a = ap.parse_args()
    for p in build_all(a.verbose, a.jobs):
        print("built", p)
