"""ctypes bindings of the CPU checkers (test infrastructure only).

`oracle()` loads liboracle.so (built by oracle/Makefile from skainet_oracle.c; built on demand if
gcc is present). `ref()` loads _ref/libskainet_ref.so -- the reference's native C kernels compiled
from the reference's own sources -- or returns None when that library was never built.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_f32p = C.POINTER(C.c_float)
_u8p = C.POINTER(C.c_uint8)
_i32p = C.POINTER(C.c_int32)
_cache: dict = {}


def fp(a):
    return None if a is None else a.ctypes.data_as(_f32p)


def u8(a):
    return a.ctypes.data_as(_u8p)


def i32(a):
    return None if a is None else a.ctypes.data_as(_i32p)


_GEMV_ARGS = [_f32p, C.c_int32, _u8p, C.c_int32, C.c_int32, C.c_int32, _f32p, C.c_int32]
_NARROW_ARGS = [_f32p, C.c_int32, C.c_int32, _u8p, C.c_int32, C.c_int32, _f32p, C.c_int32, C.c_int32] + [C.c_int32] * 3
_SDPA_ARGS = [_f32p, _f32p, _f32p, _f32p] + [C.c_int32] * 6 + [C.c_float] + [C.c_int32] * 3 + \
             [_i32p, _f32p] + [C.c_int32] * 4


def build(target: str = "liboracle.so") -> None:
    subprocess.run(["make", "-C", _DIR, target], check=True, capture_output=True)


def oracle(fast: bool = False) -> C.CDLL:
    name = "liboracle_fast.so" if fast else "liboracle.so"
    if name in _cache:
        return _cache[name]
    path = os.path.join(_DIR, name)
    if not os.path.exists(path):
        build(name)
    lib = C.CDLL(path)
    lib.orc_half_to_float.argtypes = [C.c_uint32]
    lib.orc_half_to_float.restype = C.c_float
    lib.orc_float_to_half.argtypes = [C.c_float]
    lib.orc_float_to_half.restype = C.c_uint32
    for n in ("q8_0", "q4k", "q6k", "q4_0", "q5_0", "q5_1", "q5k"):
        f = getattr(lib, f"orc_dequant_{n}")
        f.argtypes = [_u8p, C.c_int64, _f32p]
        f.restype = None
        f = getattr(lib, f"orc_{n}_matmul")
        f.argtypes = _GEMV_ARGS + [C.c_int32]
        f.restype = None
    for n in ("q8_0", "q4k", "q6k"):
        f = getattr(lib, f"orc_native_{n}_matmul_rm")
        f.argtypes = _GEMV_ARGS
        f.restype = None
    for n in ("bf16", "fp16"):
        f = getattr(lib, f"orc_{n}_matmul")
        f.argtypes = _NARROW_ARGS
        f.restype = None
    lib.orc_relayout.argtypes = [_u8p, _u8p, C.c_int64, C.c_int64, C.c_int32, C.c_int32]
    lib.orc_relayout.restype = None
    lib.orc_q8_0_quantize.argtypes = [_f32p, C.c_int64, _u8p]
    lib.orc_q8_0_quantize.restype = None
    lib.orc_f32_sdpa.argtypes = _SDPA_ARGS
    lib.orc_f32_sdpa.restype = None
    lib.orc_f32_rms_norm.argtypes = [_f32p, _f32p, _f32p, C.c_int32, C.c_int32, C.c_float]
    lib.orc_f32_rms_norm.restype = None
    lib.orc_f32_softmax_rows.argtypes = [_f32p, _f32p, C.c_int32, C.c_int32, C.c_int32]
    lib.orc_f32_softmax_rows.restype = None
    lib.orc_fp32_matmul.argtypes = [_f32p, C.c_int32, C.c_int32] * 3 + [C.c_int32] * 3
    lib.orc_fp32_matmul.restype = None
    lib.orc_fp32_matmul_wt.argtypes = [_f32p, C.c_int32] * 3 + [C.c_int32] * 3
    lib.orc_fp32_matmul_wt.restype = None
    _cache[name] = lib
    return lib


def ref():
    """The reference's own C kernels, or None when oracle/_ref was not built."""
    if "ref" in _cache:
        return _cache["ref"]
    path = os.path.join(_DIR, "_ref", "libskainet_ref.so")
    lib = None
    if os.path.exists(path):
        lib = C.CDLL(path)
        for n in ("q8_0", "q4k", "q6k", "q4_0", "q5_0", "q5_1", "q5k"):
            for suffix in ("", "_rm"):
                f = getattr(lib, f"skainet_{n}_matmul{suffix}", None)   # an older build of _ref has only the first three
                if f is not None:
                    f.argtypes = _GEMV_ARGS
                    f.restype = None
        for n in ("bf16", "fp16"):
            f = getattr(lib, f"skainet_{n}_matmul", None)
            if f is not None:
                f.argtypes = _NARROW_ARGS
                f.restype = None
        lib.skainet_f32_sdpa.argtypes = _SDPA_ARGS
        lib.skainet_f32_sdpa.restype = None
        lib.skainet_f32_rms_norm.argtypes = [_f32p, _f32p, _f32p, C.c_int32, C.c_int32, C.c_float]
        lib.skainet_f32_rms_norm.restype = None
        lib.skainet_f32_softmax_rows.argtypes = [_f32p, _f32p, C.c_int32, C.c_int32, C.c_int32]
        lib.skainet_f32_softmax_rows.restype = None
        lib.skainet_fp32_matmul.argtypes = [_f32p, C.c_int32, C.c_int32] * 3 + [C.c_int32] * 3
        lib.skainet_fp32_matmul.restype = None
        lib.skainet_fp32_matmul_wt.argtypes = [_f32p, C.c_int32] * 3 + [C.c_int32] * 3
        lib.skainet_fp32_matmul_wt.restype = None
        lib.skainet_f32_unary.argtypes = [C.c_int32, _f32p, _f32p, C.c_int32]
        lib.skainet_f32_unary.restype = None
    _cache["ref"] = lib
    return lib


# ---------------------------------------------------------------- numpy-level helpers

BLOCK = {"Q8_0": (32, 34), "Q4_K": (256, 144), "Q6_K": (256, 210), "Q4_0": (32, 18), "Q5_0": (32, 22), "Q5_1": (32, 24),
         "Q5_K": (256, 176)}
_SHORT = {"Q8_0": "q8_0", "Q4_K": "q4k", "Q6_K": "q6k", "Q4_0": "q4_0", "Q5_0": "q5_0", "Q5_1": "q5_1", "Q5_K": "q5k"}


def dequant(enc: str, w: np.ndarray) -> np.ndarray:
    bs, nb = BLOCK[enc]
    w = np.ascontiguousarray(w, dtype=np.uint8)
    blocks = w.size // nb
    out = np.empty(blocks * bs, dtype=np.float32)
    getattr(oracle(), f"orc_dequant_{_SHORT[enc]}")(u8(w), blocks, fp(out))
    return out


def gemv(enc: str, x: np.ndarray, w: np.ndarray, n: int, row_major: bool = True) -> np.ndarray:
    """Exact-fp32 y[m, n] = x[m, k] . W^T, one scalar-kernel call per activation row."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    x2 = x.reshape(-1, x.shape[-1])
    m, k = x2.shape
    w = np.ascontiguousarray(w, dtype=np.uint8)
    y = np.empty((m, n), dtype=np.float32)
    f = getattr(oracle(), f"orc_{_SHORT[enc]}_matmul")
    for r in range(m):
        f(fp(x2), r * k, u8(w), 0, k, n, fp(y), r * n, 1 if row_major else 0)
    return y.reshape(x.shape[:-1] + (n,))


def sdpa(q, k, v, scale, causal=False, window=0, right_context=0, lengths=None, mask=None, lib=None):
    """softmax(q k^T scale + rules + mask) v with the reference's argument meaning; `lib` picks the checker."""
    q = np.ascontiguousarray(q, np.float32); k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    b, h, sq, d = q.shape
    _, hkv, skv, _ = k.shape
    out = np.empty_like(q)
    md = [0, 0, 0, 0]
    if mask is not None:
        mask = np.ascontiguousarray(mask, np.float32)
        md = [1] * (4 - mask.ndim) + list(mask.shape)
    if lengths is not None:
        lengths = np.ascontiguousarray(lengths, np.int32)
    fn = oracle().orc_f32_sdpa if lib is None else lib.skainet_f32_sdpa
    fn(fp(q), fp(k), fp(v), fp(out), b, h, hkv, sq, skv, d, float(scale), int(causal), window,
       right_context, i32(lengths), fp(mask), *md)
    return out


def narrow_matmul(kind: str, a: np.ndarray, b_bytes: np.ndarray, m: int, n: int, k: int, lib=None) -> np.ndarray:
    """C(m, n) = A(m, k) B(k, n) with B as contiguous bf16 / fp16 bytes (`kind` "bf16" / "fp16"); `lib` picks the checker
    (default: the oracle; pass ref() for the reference's C library)."""
    a = np.ascontiguousarray(a, np.float32)
    b_bytes = np.ascontiguousarray(b_bytes, np.uint8)
    out = np.empty((m, n), np.float32)
    fn = getattr(oracle(), f"orc_{kind}_matmul") if lib is None else getattr(lib, f"skainet_{kind}_matmul")
    fn(fp(a), 0, k, u8(b_bytes), 0, 2 * n, fp(out), 0, n, m, n, k)
    return out
