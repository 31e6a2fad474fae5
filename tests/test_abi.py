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


def _c_parameter_kinds():
    """name -> (return kind, [parameter kinds]) of every declaration of the header; kinds are the FFM layout letters the
    Kotlin module uses: I int32, L int64 / size_t, F float, P pointer, V void."""
    text = open(os.path.join(ROOT, "include", "skainet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)

    def kind(decl):
        decl = decl.strip()
        if "*" in decl:
            return "P"
        base = decl.split()
        if not base or decl == "void":
            return "V"
        if "float" in base:
            return "F"
        if "int64_t" in base or "size_t" in base:
            return "L"
        if "int32_t" in base:
            return "I"
        raise AssertionError(f"unclassified C type in {decl!r}")

    out = {}
    for m in re.finditer(r"SKAINET_HIP_API\s+([^;]*?)\b(skainet_hip_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        ret, name, params = m.group(1), m.group(2), m.group(3)
        plist = [] if params.strip() in ("", "void") else [kind(p) for p in params.split(",")]
        out[name] = (kind(ret + " x") if "*" in ret else kind(ret), plist)
    return out


def test_kotlin_module_binds_the_header_as_declared():
    """The Kotlin module text is not compiled here, so its native descriptors are held against the header: every symbol
    it binds is declared, with the same return and parameter layouts; both ServiceLoader files name classes that exist."""
    kdir = os.path.join(ROOT, "kotlin", "skainet-backend-hip", "src", "jvmMain")
    src = open(os.path.join(kdir, "kotlin", "sk", "ainet", "exec", "hip", "HipLibrary.kt")).read()
    decls = _c_parameter_kinds()
    named = {m.group(1): m.group(2) for m in re.finditer(r"private val (\w+): FunctionDescriptor = (FunctionDescriptor\.\w+\([^)]*\))", src)}
    bound = re.findall(r'bind\(\s*"(skainet_hip_\w+)",\s*(FunctionDescriptor\.\w+\([^)]*\)|\w+)', src)
    assert len(bound) >= 39
    for name, desc in bound:
        assert name in decls, f"{name} is not declared in the header"
        desc = named.get(desc, desc)
        m = re.match(r"FunctionDescriptor\.(of|ofVoid)\(([^)]*)\)", desc)
        assert m, (name, desc)
        letters = [t.strip() for t in m.group(2).split(",") if t.strip()]
        ret, params = ("V", letters) if m.group(1) == "ofVoid" else (letters[0], letters[1:])
        assert (ret, params) == decls[name], (name, ret, params, decls[name])
    all_kt = "".join(open(os.path.join(kdir, "kotlin", "sk", "ainet", "exec", "hip", f)).read()
                     for f in sorted(os.listdir(os.path.join(kdir, "kotlin", "sk", "ainet", "exec", "hip"))))
    assert "TODO" not in all_kt
    services = os.path.join(kdir, "resources", "META-INF", "services")
    for iface in ("sk.ainet.backend.api.kernel.KernelProvider", "sk.ainet.backend.api.kernel.ViewKernelPack"):
        cls = open(os.path.join(services, iface)).read().strip()
        assert cls.startswith("sk.ainet.exec.hip.") and f"class {cls.rsplit('.', 1)[1]} " in all_kt
    # every accessor of the provider interface the Python mirror serves is served by the Kotlin provider as well
    provider = open(os.path.join(kdir, "kotlin", "sk", "ainet", "exec", "hip", "HipKernelProvider.kt")).read()
    for accessor in ("matmulFp32", "matmulFp32Wt", "matmulBf16", "matmulFp16", "matmulQ4K", "matmulQ6K", "matmulQ5K", "matmulQ8_0",
                     "matmulQ4_0", "matmulQ5_0", "matmulQ5_1", "softmaxFp32", "normFp32", "attentionFp32"):
        assert f"override fun {accessor}()" in provider


def test_resident_ops_class_serves_the_reference_method_set_in_both_languages():
    """The resident-activation ops class overrides the methods the browser tier's resident ops class overrides
    (WasmCpuOps.kt:180-428: the two matmuls, four binaries, six activations, two reductions, softmax / logSoftmax, the two
    fused norms, attention) -- in the Kotlin text and in the Python mirror that the GPU tests drive -- and every device
    entry the Kotlin class calls is bound in HipLibrary.kt (whose descriptors the test above holds against the header)."""
    kdir = os.path.join(ROOT, "kotlin", "skainet-backend-hip", "src", "jvmMain", "kotlin", "sk", "ainet", "exec", "hip")
    ops_kt = open(os.path.join(kdir, "HipOps.kt")).read()
    lib_kt = open(os.path.join(kdir, "HipLibrary.kt")).read()
    methods = ["matmul", "matmulWeightTransposed", "add", "subtract", "multiply", "divide", "relu", "sigmoid", "silu", "gelu",
               "erf", "tanh", "sum", "mean", "softmax", "logSoftmax", "layerNorm", "rmsNorm", "scaledDotProductAttention"]
    from skainet_amd import ops as py_ops
    for name in methods:
        assert re.search(r"override fun <T : DType, V> %s\(" % name, ops_kt), f"HipOps.kt does not override {name}"
        snake = re.sub(r"(?<!^)(?=[A-Z])", "_", name).lower()
        assert callable(getattr(py_ops.HipOps, snake, None)), f"ops.HipOps has no {snake}"
    assert "fun <T : DType, V> toResident(" in ops_kt and callable(py_ops.HipOps.to_resident)
    for handle in set(re.findall(r"HipLibrary\.(\w+)", ops_kt)):
        assert re.search(r"\b(val|fun) %s\b" % handle, lib_kt), f"HipLibrary has no member {handle}"
    assert "class HipTensorData" in open(os.path.join(kdir, "HipTensorData.kt")).read()


def test_no_alloc_argmax_hands_each_host_thread_a_slot_of_its_own():
    """The arg-max entry that allocates nothing keeps its counters in a fixed array cut into 8 slots; a host thread gets
    one on first use and keeps it (the library's streams are per thread). The hand-out makes no device call, so it is
    checked here, in a fresh process: ten threads, each asking twice -- eight distinct slots 0..7, the same slot on the
    second call, -1 for the two that come too late."""
    import subprocess
    import sys
    code = (
        "import ctypes, threading, sys\n"
        f"lib = ctypes.CDLL({_lib.HIP_LIB_PATH!r})\n"
        "f = lib.skainet_hip_f32_argmax_rows_noalloc_slot; f.restype = ctypes.c_int32\n"
        "out = [None] * 10\n"
        "gate = threading.Barrier(10)\n"
        "def work(i):\n"
        "    gate.wait(); a = f(); b = f(); gate.wait(); out[i] = (a, b)\n"
        "ts = [threading.Thread(target=work, args=(i,)) for i in range(10)]\n"
        "[t.start() for t in ts]; [t.join() for t in ts]\n"
        "print(sorted(out))\n")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    got = eval(r.stdout.strip())
    assert all(a == b for a, b in got)                                       # a thread keeps its slot
    assert sorted(a for a, _ in got) == [-1, -1] + list(range(8))            # eight slots, then refusals
