"""The C-ABI library loads and exports every symbol include/skainet_hip.h declares; without a GPU it answers
"unavailable" and the product path fails loudly instead of falling back to anything on the CPU."""
import ctypes
import os
import re

import numpy as np
import pytest

from skainet_amd import _lib, kernels

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "skainet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(skainet_hip_\w+)\s*\(", text)))


def test_header_and_binding_table_agree():
    names = declared_symbols()
    assert len(names) >= 40
    assert sorted(_lib.SIGNATURES) == names


@pytest.mark.parametrize("compiler,lang", [("gcc", "c"), ("g++", "c++")])
def test_header_is_plain_c_and_cpp(compiler, lang, tmp_path):
    """The boundary is a C ABI: the header compiles on its own as C and as C++ (no torch or HIP types in it), and a
    program written against it links with nothing but the shared library."""
    import shutil
    import subprocess
    if shutil.which(compiler) is None:
        pytest.skip(f"{compiler} not installed")
    src = tmp_path / ("use." + ("c" if lang == "c" else "cpp"))
    src.write_text('#include "skainet_hip.h"\n#include <stdio.h>\n'
                   'int main(void) { printf("%d\\n", (int)skainet_hip_available()); return 0; }\n')
    exe = tmp_path / "use"
    pkg = os.path.dirname(_lib.HIP_LIB_PATH)
    r = subprocess.run([compiler, "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
                        "-L", pkg, "-lskainet_hip", f"-Wl,-rpath,{pkg}"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0 and run.stdout.strip() in ("0", "1"), (run.stdout, run.stderr)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.HIP_LIB_PATH)
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, missing


def test_quantizer_library_exports():
    lib = ctypes.CDLL(_lib.QUANT_LIB_PATH)
    for n in ("skainet_quantize_q8_0", "skainet_quantize_q4k", "skainet_quantize_q6k", "skainet_quantize_q4_0",
              "skainet_quantize_q5_0", "skainet_quantize_q5_1", "skainet_quantize_q5k"):
        assert hasattr(lib, n)


def _no_gpu():
    import torch
    return not torch.cuda.is_available()


@pytest.mark.skipif(not _no_gpu(), reason="exercises the no-device contract")
def test_unavailable_is_an_answer_and_calls_fail_loudly():
    assert kernels.is_available() is False          # cached, no exception (KernelProvider.isAvailable contract)
    provider = kernels.HipKernelProvider()
    assert provider.name == "hip" and provider.priority > kernels.PRIORITY_NATIVE
    assert provider.matmul_q4k() is None and provider.attention_fp32() is None
    assert provider.supports("matmul", ["Float32", "Q4_K"]) is False
    k = kernels.HipPackedMatmulKernel("Q4_K")
    x, w, y = np.zeros(256, np.float32), np.zeros(144 * 2, np.uint8), np.zeros(2, np.float32)
    with pytest.raises(kernels.HipError):            # IllegalStateException analogue: never a silent CPU result
        k.matmul(x, 0, w, 0, 256, 2, y, 0)
    with pytest.raises(ValueError):                  # IllegalArgumentException analogue comes first
        k.matmul(x, 0, w, 0, 100, 2, y, 0)
    with pytest.raises(kernels.HipError):
        kernels.DeviceWeight.upload("Q4_K", w, 2, 256)
    # the raw C entry leaves the output untouched and says why
    y[:] = 7
    _lib.hip().skainet_hip_q4k_matmul_rm(x.ctypes.data, 0, w.ctypes.data, 0, 256, 2, y.ctypes.data, 0)
    assert (y == 7).all() and _lib.last_error()
