"""ctypes binding of libskainet_hip.so (the C ABI in include/skainet_hip.h) and libskainet_quant.so.

The product path has no CPU fallback: `hip()` raises when the library is missing, and every wrapper in
`skainet_amd.kernels` raises `HipError` when a device call fails.
"""
from __future__ import annotations

import ctypes as C
import importlib.util
import os
import sys

_PKG = os.path.dirname(os.path.abspath(__file__))
_vp, _i32, _i64, _f32, _sz = C.c_void_p, C.c_int32, C.c_int64, C.c_float, C.c_size_t

_GEMV = [_vp, _i32, _vp, _i32, _i32, _i32, _vp, _i32]
_SGEMM = [_vp, _i32, _i32] * 3 + [_i32] * 3
_SGEMM_WT = [_vp, _i32] * 3 + [_i32] * 3
_SDPA = [_vp] * 4 + [_i32] * 6 + [_f32] + [_i32] * 3 + [_vp, _vp] + [_i32] * 4

# name -> (restype, argtypes); mirrors include/skainet_hip.h one to one
SIGNATURES = {
    "skainet_hip_available": (_i32, []),
    "skainet_hip_init": (_i32, [_i32]),
    "skainet_hip_last_error": (C.c_char_p, []),
    "skainet_hip_device_name": (C.c_char_p, []),
    "skainet_hip_compute_units": (_i32, []),
    "skainet_hip_last_kernel": (C.c_char_p, []),
    "skainet_hip_set_stream": (_i32, [_vp]),
    "skainet_hip_thread_stream": (_i32, []),
    "skainet_hip_sync": (_i32, []),
    "skainet_hip_thread_release": (_i32, []),
    "skainet_hip_malloc": (_vp, [_sz]),
    "skainet_hip_free": (_i32, [_vp]),
    "skainet_hip_memcpy_h2d": (_i32, [_vp, _vp, _sz]),
    "skainet_hip_memcpy_d2h": (_i32, [_vp, _vp, _sz]),
    "skainet_hip_memcpy_d2d": (_i32, [_vp, _vp, _sz]),
    "skainet_hip_host_alloc": (_vp, [_sz]),
    "skainet_hip_host_free": (_i32, [_vp]),
    "skainet_hip_timer_begin": (_i32, []),
    "skainet_hip_timer_end_ms": (_f32, []),
    "skainet_hip_weight_upload": (_vp, [_vp, _i64, _i32, _i32, _i32, _i32]),
    "skainet_hip_weight_wrap": (_vp, [_vp, _i32, _i32, _i32]),
    "skainet_hip_weight_free": (None, [_vp]),
    "skainet_hip_weight_data": (_vp, [_vp]),
    "skainet_hip_weight_nbytes": (_i64, [_vp]),
    "skainet_hip_matmul_dev": (_i32, [_vp, _vp, _i32, _vp]),
    "skainet_hip_matmul_host": (_i32, [_vp, _vp, _i32, _vp]),
    "skainet_hip_matmul_kind_dev": (_i32, [_vp, _vp, _i32, _vp, _i32]),
    "skainet_hip_matmul_fused_dev": (_i32, [_vp, _vp, _i32, _vp, _vp, _f32, _vp, _i32]),
    "skainet_hip_matmul_qkv_rope_dev": (_i32, [_vp, _vp, _vp, _f32, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp, _f32, _vp]),
    "skainet_hip_f32_rope_table_dev": (_i32, [_vp, _f32, _i32, _vp]),
    "skainet_hip_matmul_repeat_dev": (_f32, [_vp, _i32, _vp, _i32, _vp, _i32, _i32, _i32, _i32]),
    "skainet_hip_read_probe_dev": (_f32, [_vp, _i32, _i64, _i32, _i32]),
    "skainet_hip_dequantize_dev": (_i32, [_vp, _vp]),
    "skainet_hip_dequantize_rows_dev": (_i32, [_vp, _vp, _i32, _vp]),
    "skainet_hip_q4k_matmul": (None, _GEMV),
    "skainet_hip_q4k_matmul_rm": (None, _GEMV),
    "skainet_hip_q6k_matmul": (None, _GEMV),
    "skainet_hip_q6k_matmul_rm": (None, _GEMV),
    "skainet_hip_q8_0_matmul": (None, _GEMV),
    "skainet_hip_q8_0_matmul_rm": (None, _GEMV),
    "skainet_hip_q4_0_matmul": (None, _GEMV),
    "skainet_hip_q4_0_matmul_rm": (None, _GEMV),
    "skainet_hip_q5_0_matmul": (None, _GEMV),
    "skainet_hip_q5_0_matmul_rm": (None, _GEMV),
    "skainet_hip_q5_1_matmul": (None, _GEMV),
    "skainet_hip_q5_1_matmul_rm": (None, _GEMV),
    "skainet_hip_q5k_matmul": (None, _GEMV),
    "skainet_hip_q5k_matmul_rm": (None, _GEMV),
    "skainet_hip_fp32_matmul": (None, _SGEMM),
    "skainet_hip_fp32_matmul_wt": (None, _SGEMM_WT),
    "skainet_hip_bf16_matmul": (None, _SGEMM),
    "skainet_hip_fp16_matmul": (None, _SGEMM),
    "skainet_hip_f32_rms_norm": (None, [_vp, _vp, _vp, _i32, _i32, _f32]),
    "skainet_hip_f32_layer_norm": (None, [_vp, _vp, _vp, _vp, _i32, _i32, _f32]),
    "skainet_hip_f32_softmax_rows": (None, [_vp, _vp, _i32, _i32, _i32]),
    "skainet_hip_f32_sdpa": (None, _SDPA),
    "skainet_hip_fp32_matmul_dev": (_i32, _SGEMM),
    "skainet_hip_fp32_matmul_wt_dev": (_i32, _SGEMM_WT),
    "skainet_hip_f32_rms_norm_dev": (_i32, [_vp, _vp, _vp, _i32, _i32, _f32]),
    "skainet_hip_f32_layer_norm_dev": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _f32]),
    "skainet_hip_f32_softmax_rows_dev": (_i32, [_vp, _vp, _i32, _i32, _i32]),
    "skainet_hip_f32_sdpa_dev": (_i32, _SDPA),
    "skainet_hip_f32_binary_dev": (_i32, [_i32, _vp, _i32, _vp, _i32, _vp, _i64, _i32]),
    "skainet_hip_f32_unary_dev": (_i32, [_i32, _vp, _vp, _i64]),
    "skainet_hip_f32_reduce_all_dev": (_i32, [_vp, _i64, _i32, _vp]),
    "skainet_hip_f32_reduce_axis_dev": (_i32, [_vp, _i32, _i32, _i32, _i32, _vp]),
    "skainet_hip_mlp_swiglu_dev": (_i32, [_vp, _vp, _vp, _i32, _vp, _f32, _vp, _vp]),
    "skainet_hip_attn_out_proj_dev": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp, _vp, _vp, _vp]),
    "skainet_hip_f32_sdpa_cache_dev": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _i32, _i32,
                                              _vp]),
    "skainet_hip_f32_sdpa_cache_rows_dev": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _i32,
                                                   _i32, _vp]),
    "skainet_hip_f32_silu_mul_dev": (_i32, [_vp, _vp, _vp, _i64]),
    "skainet_hip_f32_add_dev": (_i32, [_vp, _vp, _vp, _i64]),
    "skainet_hip_f32_argmax_rows_dev": (_i32, [_vp, _i32, _i32, _vp]),
    "skainet_hip_f32_argmax_rows_noalloc_dev": (_i32, [_vp, _i32, _i32, _vp]),
    "skainet_hip_f32_argmax_rows_noalloc_slot": (_i32, []),
    "skainet_hip_f32_rope_scatter_dev": (_i32, [_vp, _i64, _vp, _i32, _i32, _i32, _i32, _vp, _f32, _i32, _i64, _i32]),
    "skainet_hip_decode_advance_dev": (_i32, [_vp, _vp, _vp, _vp, _i32]),
    "skainet_hip_i32_store_at_dev": (_i32, [_vp, _vp, _i32, _vp]),
    "skainet_hip_f32_swiglu_pairs_dev": (_i32, [_vp, _vp, _i64]),
    "skainet_hip_f32_rope_qkv_dev": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _vp, _f32]),
    "skainet_hip_f32_heads_to_rows_dev": (_i32, [_vp, _vp, _i32, _i32, _i32]),
    "skainet_hip_i32_increment_dev": (_i32, [_vp, _i32]),
    "skainet_hip_graph_begin": (_i32, []),
    "skainet_hip_graph_end": (_vp, []),
    "skainet_hip_graph_launch": (_i32, [_vp]),
    "skainet_hip_graph_valid": (_i32, [_vp]),
    "skainet_hip_graph_sync": (_i32, [_vp]),
    "skainet_hip_graph_free": (None, [_vp]),
    "skainet_hip_set_tuning": (_i32, [C.c_char_p, _i32]),
}

HIP_LIB_PATH = os.path.join(_PKG, "libskainet_hip.so")
QUANT_LIB_PATH = os.path.join(_PKG, "libskainet_quant.so")
_hip = None
_quant = None


class HipError(RuntimeError):
    """A device call failed, or the HIP library / a gfx950 device is missing."""


def _share_hip_runtime_with_torch() -> None:
    """One HIP runtime per process: PyTorch wheels carry their own libamdhip64.so.7, and the dynamic loader hands
    whichever copy was loaded first to every later client of that soname. When torch is installed, load ITS copy
    before this library so that device pointers, streams and the device count agree whichever is imported first
    (with the system copy loaded first, torch reports no GPU). Without torch the system runtime is used."""
    if "torch" in sys.modules:
        return
    try:
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        spec = None
    for loc in (spec.submodule_search_locations if spec and spec.submodule_search_locations else []):
        path = os.path.join(loc, "lib", "libamdhip64.so")
        if os.path.exists(path):
            try:
                C.CDLL(path, mode=C.RTLD_GLOBAL)
            except OSError:
                pass
            return


def hip() -> C.CDLL:
    """The loaded kernel library. Raises HipError when it was not built (python -m skainet_amd.build)."""
    global _hip
    if _hip is None:
        if not os.path.exists(HIP_LIB_PATH):
            raise HipError(f"{HIP_LIB_PATH} is missing: build it with `python -m skainet_amd.build`")
        _share_hip_runtime_with_torch()
        lib = C.CDLL(HIP_LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _hip = lib
    return _hip


def quant() -> C.CDLL:
    global _quant
    if _quant is None:
        if not os.path.exists(QUANT_LIB_PATH):
            raise HipError(f"{QUANT_LIB_PATH} is missing: build it with `python -m skainet_amd.build`")
        lib = C.CDLL(QUANT_LIB_PATH)
        for n in ("q8_0", "q4k", "q6k", "q4_0", "q5_0", "q5_1", "q5k"):
            fn = getattr(lib, f"skainet_quantize_{n}")
            fn.restype, fn.argtypes = None, [_vp, _i64, _vp]
        _quant = lib
    return _quant


def last_error() -> str:
    return hip().skainet_hip_last_error().decode("utf-8", "replace")


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise HipError(f"{what}: {last_error()}")
