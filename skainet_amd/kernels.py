"""Host-side mirror of the reference's kernel SPI for the HIP backend.

Same names, argument meaning and error behaviour as `skainet-backend-api`
(/root/reference/skainet-backends/skainet-backend-api/src/commonMain/kotlin/sk/ainet/backend/api/kernel/):

    KernelProvider.kt:22-190      -> HipKernelProvider (name, priority, is_available, matmul_q4k(), ...)
    Q4KMatmulKernel.kt:43-72      -> HipPackedMatmulKernel.matmul(input, input_offset, weight, weight_byte_offset,
    Q6KMatmulKernel.kt:33           input_dim, output_dim, output, output_offset): weight input-block-major,
    Q8_0MatmulKernel.kt:31          input_dim % block_size != 0 -> ValueError (IllegalArgumentException),
                                    backend unavailable at call time -> HipError (IllegalStateException)
    Fp32MatmulKernel.kt:25-50     -> HipFp32MatmulKernel.matmul
    Fp32MatmulWtKernel.kt:21-28   -> HipFp32MatmulWtKernel.matmul_wt
    Fp32FusedKernels.kt:15,37,75  -> HipFp32SoftmaxKernel / HipFp32NormKernel / HipFp32AttentionKernel
    MatmulKernels.kt:11-40        -> HipRowMajorMatmulKernel.run (the ViewKernel for GGUF-ordered weights:
                                    all activation rows at once, weight resident on the device)

The JVM arrays of the SPI are numpy arrays here; every call goes through the C ABI of libskainet_hip.so
(skainet_amd._lib). Device-resident operation (weights uploaded once, activations staying on the GPU) is
`DeviceWeight` plus the `*_dev` functions, which take raw device addresses (e.g. torch's `.data_ptr()`).
"""
from __future__ import annotations

import ctypes as C
import threading
from typing import Optional

import numpy as np

from . import _lib
from ._lib import HipError, check

# TensorEncoding.name -> (C ABI id, block elements, bytes per block)
ENCODINGS = {"Q8_0": (8, 32, 34), "Q4_K": (12, 256, 144), "Q6_K": (14, 256, 210),
             "Q4_0": (2, 32, 18), "Q5_0": (6, 32, 22), "Q5_1": (7, 32, 24), "Q5_K": (13, 256, 176)}
ORDER_ROW_MAJOR, ORDER_INPUT_BLOCK_MAJOR = 0, 1

PRIORITY_SCALAR, PRIORITY_PANAMA, PRIORITY_NATIVE = 0, 50, 100   # KernelProvider.kt:15-17
PRIORITY_HIP = 200


def _ptr(a) -> int:
    """Address of a numpy array, a torch tensor, or an int that already is an address; None -> 0."""
    if a is None:
        return 0
    if isinstance(a, int):
        return a
    if isinstance(a, np.ndarray):
        return a.ctypes.data
    return a.data_ptr()


def _f32(a, name) -> np.ndarray:
    if not isinstance(a, np.ndarray) or a.dtype != np.float32 or not a.flags.c_contiguous:
        raise TypeError(f"{name} must be a C-contiguous float32 numpy array")
    return a


def _require_available() -> None:
    if not is_available():
        raise HipError("HIP backend unavailable: " + _lib.last_error())


_avail_lock = threading.Lock()
_avail: Optional[bool] = None


def is_available() -> bool:
    """Cheap, cached, never raises: False when the library or a gfx950 device is missing."""
    global _avail
    if _avail is None:
        with _avail_lock:
            if _avail is None:
                try:
                    _avail = bool(_lib.hip().skainet_hip_available())
                except (HipError, OSError):
                    _avail = False
    return _avail


# ---------------------------------------------------------------------------------------------- quantizers

def quantize(encoding: str, values: np.ndarray) -> np.ndarray:
    """fp32 values (size a multiple of the block size, blocks along the last axis) -> packed row-major bytes.

    Q8_0 follows Q8_0Quantizer.quantizeToBytes
    (/root/reference/skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/data/Q8_0Quantizer.kt:28-53);
    Q4_0 follows Q4_0Quantizer.quantizeToBytes (same directory, Q4_0Quantizer.kt:28-66);
    Q4_K / Q6_K / Q5_K / Q5_0 / Q5_1 follow the ggml reference quantizers (the reference has none for them).
    """
    _, bs, nb = ENCODINGS[encoding]
    v = np.ascontiguousarray(values, dtype=np.float32)
    if v.size % bs != 0 or (v.ndim > 0 and v.shape[-1] % bs != 0):
        raise ValueError(f"{encoding} quantization requires a last dimension that is a multiple of {bs}; got {v.shape}")
    out = np.empty(v.size // bs * nb, dtype=np.uint8)
    fn = getattr(_lib.quant(), {"Q8_0": "skainet_quantize_q8_0", "Q4_K": "skainet_quantize_q4k", "Q6_K": "skainet_quantize_q6k",
                                "Q4_0": "skainet_quantize_q4_0", "Q5_0": "skainet_quantize_q5_0",
                                "Q5_1": "skainet_quantize_q5_1", "Q5_K": "skainet_quantize_q5k"}[encoding])
    fn(v.ctypes.data, v.size, out.ctypes.data)
    return out


def to_kernel_order(encoding: str, row_major: np.ndarray, rows: int, blocks_per_row: int) -> np.ndarray:
    """PackedWeights.toKernelOrder (PackedWeights.kt:63-93): kernel[(b*rows+o)] = canonical[(o*bpr+b)], block-wise."""
    nb = ENCODINGS[encoding][2]
    return np.ascontiguousarray(
        row_major.reshape(rows, blocks_per_row, nb).transpose(1, 0, 2)).reshape(-1)


# ---------------------------------------------------------------------------------------------- device weights

EPI_NONE, EPI_RESIDUAL, EPI_SWIGLU = 0, 1, 2


class PinnedBytes:
    """Page-locked host bytes from the library (skainet_hip_host_alloc) as a numpy uint8 array: read a weight file into
    `.array` and DeviceWeight.upload moves it in one DMA transfer. The memory lives until close() / garbage collection;
    `.array` must not be used afterwards."""

    def __init__(self, nbytes: int):
        _require_available()
        self.nbytes = int(nbytes)
        self.ptr = _lib.hip().skainet_hip_host_alloc(self.nbytes)
        if not self.ptr:
            raise HipError("host_alloc: " + _lib.last_error())
        self.array = np.ctypeslib.as_array((C.c_uint8 * max(self.nbytes, 1)).from_address(self.ptr))[: self.nbytes]

    def close(self) -> None:
        if self.ptr:
            self.array = None
            _lib.hip().skainet_hip_host_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class DeviceWeight:
    """A packed [rows, cols] weight resident on the device (canonical row-major blocks)."""

    def __init__(self, handle: int, encoding: str, rows: int, cols: int, keepalive=None):
        self._h, self.encoding, self.rows, self.cols = handle, encoding, rows, cols
        self._keepalive = keepalive

    @classmethod
    def upload(cls, encoding: str, packed: np.ndarray, rows: int, cols: int, order: int = ORDER_ROW_MAJOR) -> "DeviceWeight":
        _require_available()
        enc_id, bs, nb = ENCODINGS[encoding]
        if cols % bs != 0:
            raise ValueError(f"inputDim must be a multiple of {bs}; got {cols}")
        packed = np.ascontiguousarray(packed, dtype=np.uint8)
        h = _lib.hip().skainet_hip_weight_upload(packed.ctypes.data, packed.size, enc_id, order, rows, cols)
        if not h:
            raise HipError("weight_upload: " + _lib.last_error())
        return cls(h, encoding, rows, cols)

    @classmethod
    def wrap(cls, encoding: str, device_bytes, rows: int, cols: int) -> "DeviceWeight":
        """View packed row-major bytes already on the device (`device_bytes`: tensor or address); not owned."""
        _require_available()
        h = _lib.hip().skainet_hip_weight_wrap(_ptr(device_bytes), ENCODINGS[encoding][0], rows, cols)
        if not h:
            raise HipError("weight_wrap: " + _lib.last_error())
        return cls(h, encoding, rows, cols, keepalive=device_bytes)

    @property
    def nbytes(self) -> int:
        return _lib.hip().skainet_hip_weight_nbytes(self._h)

    @property
    def data_ptr(self) -> int:
        return _lib.hip().skainet_hip_weight_data(self._h)

    def matmul(self, x, m: int, out, kind: Optional[int] = None) -> None:
        """out[m, rows] = x[m, cols] . W^T on device buffers; kind None = auto, 0 = GEMV path, 1 = MFMA GEMM path."""
        if kind is None:
            check(_lib.hip().skainet_hip_matmul_dev(self._h, _ptr(x), m, _ptr(out)), "matmul")
        else:
            check(_lib.hip().skainet_hip_matmul_kind_dev(self._h, _ptr(x), m, _ptr(out), kind), "matmul")

    def matmul_host(self, a: np.ndarray, out: np.ndarray) -> None:
        """out[m, rows] = a[m, cols] . W^T with host arrays on both sides (skainet_hip_matmul_host): one upload, one
        launch chain, one download, one wait, all on buffers the calling thread re-uses."""
        a, out = _f32(a, "a"), _f32(out, "out")
        if a.ndim != 2 or a.shape[1] != self.cols or out.shape != (a.shape[0], self.rows):
            raise ValueError(f"matmul_host: a {a.shape} x W [{self.rows}, {self.cols}] -> out {out.shape} do not fit")
        check(_lib.hip().skainet_hip_matmul_host(self._h, a.ctypes.data, a.shape[0], out.ctypes.data), "matmul_host")

    def matmul_fused(self, x, m: int, out, gain=None, eps: float = 0.0, residual=None, epilogue: int = 0) -> None:
        """out = epilogue(W . rmsnorm(x) if gain is given else W . x); epilogue EPI_NONE / EPI_RESIDUAL / EPI_SWIGLU."""
        check(_lib.hip().skainet_hip_matmul_fused_dev(self._h, _ptr(x), m, _ptr(out), _ptr(gain), eps, _ptr(residual), epilogue),
              "matmul_fused")

    def matmul_qkv_rope(self, x, q_out, k_cache, v_cache, heads, kv_heads, head_dim, kv_capacity, pos_dev, theta,
                        gain=None, eps: float = 0.0, rope_table=None) -> None:
        """One token's [q | k | v] projection + RoPE + cache append (skainet_hip_matmul_qkv_rope_dev)."""
        check(_lib.hip().skainet_hip_matmul_qkv_rope_dev(self._h, _ptr(x), _ptr(gain), eps, _ptr(q_out), _ptr(k_cache),
                                                         _ptr(v_cache), heads, kv_heads, head_dim, kv_capacity,
                                                         _ptr(pos_dev), theta, _ptr(rope_table)), "matmul_qkv_rope")

    def attn_out_proj(self, q, k_cache, v_cache, heads, kv_heads, head_dim, seq_kv, kv_capacity, scale, out, attn_tmp,
                      residual=None, window: int = 0, lengths=None) -> None:
        """out = (residual or 0) + W . sdpa(q, cache) for one decode token (skainet_hip_attn_out_proj_dev)."""
        check(_lib.hip().skainet_hip_attn_out_proj_dev(self._h, _ptr(q), _ptr(k_cache), _ptr(v_cache), heads, kv_heads, head_dim,
                                                       seq_kv, kv_capacity, scale, window, _ptr(lengths), _ptr(residual),
                                                       _ptr(out), _ptr(attn_tmp)), "attn_out_proj")

    def mlp_swiglu(self, w_down: "DeviceWeight", x, m: int, out, gain=None, eps: float = 0.0, residual=None) -> None:
        """self holds interleaved (gate, up) rows: out = (residual or 0) + Wdown . swiglu(self . rmsnorm(x))
        (skainet_hip_mlp_swiglu_dev)."""
        check(_lib.hip().skainet_hip_mlp_swiglu_dev(self._h, w_down._h, _ptr(x), m, _ptr(gain), eps, _ptr(residual), _ptr(out)),
              "mlp_swiglu")

    def dequantize(self, out) -> None:
        check(_lib.hip().skainet_hip_dequantize_dev(self._h, _ptr(out)), "dequantize")

    def dequantize_rows(self, row_ids, count: int, out) -> None:
        check(_lib.hip().skainet_hip_dequantize_rows_dev(self._h, _ptr(row_ids), count, _ptr(out)), "dequantize_rows")

    def close(self) -> None:
        if self._h:
            _lib.hip().skainet_hip_weight_free(self._h)
            self._h = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def matmul_repeat(weights, x, m: int, out, iters: int, kind: int = 0, use_graph: bool = True, replays: int = 1) -> float:
    """Time `iters` back-to-back products rotating over `weights` (DeviceWeight list); returns the milliseconds of one
    pass (the median of `replays` timed passes)."""
    arr = (C.c_void_p * len(weights))(*[w._h for w in weights])
    ms = _lib.hip().skainet_hip_matmul_repeat_dev(arr, len(weights), _ptr(x), m, _ptr(out), iters, kind, int(use_graph), replays)
    if ms < 0:
        raise HipError("matmul_repeat: " + _lib.last_error())
    return ms


# ---------------------------------------------------------------------------------------------- device ops

def read_probe(buffers, nbytes: int, iters: int, grid: int = 0) -> float:
    """Milliseconds for `iters` launches of the pure streaming-read kernel rotating over `buffers` (device addresses/tensors)."""
    arr = (C.c_void_p * len(buffers))(*[_ptr(b) for b in buffers])
    ms = _lib.hip().skainet_hip_read_probe_dev(arr, len(buffers), nbytes, iters, grid)
    if ms < 0:
        raise HipError("read_probe: " + _lib.last_error())
    return ms


def last_kernel() -> str:
    """Kernel family the calling thread's last matmul / attention entry launched as its main kernel."""
    return _lib.hip().skainet_hip_last_kernel().decode()


def set_tuning(key: str, value: int) -> None:
    """Launch-shape / kernel-variant knob of the library (skainet_hip_set_tuning); unknown keys raise."""
    check(_lib.hip().skainet_hip_set_tuning(key.encode(), int(value)), "set_tuning")


def sync() -> None:
    check(_lib.hip().skainet_hip_sync(), "sync")


def thread_release() -> None:
    """Give the calling thread's library scratch back to the device (skainet_hip_thread_release): for worker threads
    that end before the process does. Graphs recorded on this thread must be freed first."""
    check(_lib.hip().skainet_hip_thread_release(), "thread_release")


def rms_norm_dev(x, gamma, out, rows: int, cols: int, eps: float) -> None:
    check(_lib.hip().skainet_hip_f32_rms_norm_dev(_ptr(x), _ptr(gamma), _ptr(out), rows, cols, eps), "rms_norm")


def layer_norm_dev(x, gamma, beta, out, rows: int, cols: int, eps: float) -> None:
    check(_lib.hip().skainet_hip_f32_layer_norm_dev(_ptr(x), _ptr(gamma), _ptr(beta), _ptr(out), rows, cols, eps), "layer_norm")


def softmax_rows_dev(x, out, rows: int, cols: int, log: bool = False) -> None:
    check(_lib.hip().skainet_hip_f32_softmax_rows_dev(_ptr(x), _ptr(out), rows, cols, int(log)), "softmax_rows")


def sdpa_dev(q, k, v, out, batch, heads, kv_heads, seq_q, seq_kv, head_dim, scale, causal=False, window=0,
             right_context=0, key_lengths=None, mask=None, mask_dims=(0, 0, 0, 0)) -> None:
    check(_lib.hip().skainet_hip_f32_sdpa_dev(_ptr(q), _ptr(k), _ptr(v), _ptr(out), batch, heads, kv_heads, seq_q, seq_kv,
                                              head_dim, scale, int(causal), window, right_context, _ptr(key_lengths),
                                              _ptr(mask), *mask_dims), "sdpa")


def sdpa_cache_dev(q, k_cache, v_cache, out, batch, heads, kv_heads, seq_q, seq_kv, kv_capacity, head_dim, scale,
                   causal=False, window=0, right_context=0, key_lengths=None) -> None:
    """SDPA over K / V stored [batch, kv_heads, kv_capacity, head_dim] of which the first seq_kv rows are keys."""
    check(_lib.hip().skainet_hip_f32_sdpa_cache_dev(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), batch, heads, kv_heads,
                                                    seq_q, seq_kv, kv_capacity, head_dim, scale, int(causal), window,
                                                    right_context, _ptr(key_lengths)), "sdpa_cache")


def sdpa_cache_rows_dev(q, k_cache, v_cache, out, batch, heads, kv_heads, seq_q, seq_kv, kv_capacity, head_dim, scale,
                        causal=False, window=0, right_context=0, key_lengths=None) -> None:
    """sdpa_cache_dev with the output as token rows, [batch, seq_q, heads, head_dim] (skainet_hip_f32_sdpa_cache_rows_dev)."""
    check(_lib.hip().skainet_hip_f32_sdpa_cache_rows_dev(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), batch, heads, kv_heads,
                                                         seq_q, seq_kv, kv_capacity, head_dim, scale, int(causal), window,
                                                         right_context, _ptr(key_lengths)), "sdpa_cache_rows")


def silu_mul_dev(gate, up, out, n: int) -> None:
    check(_lib.hip().skainet_hip_f32_silu_mul_dev(_ptr(gate), _ptr(up), _ptr(out), n), "silu_mul")


def add_dev(a, b, out, n: int) -> None:
    check(_lib.hip().skainet_hip_f32_add_dev(_ptr(a), _ptr(b), _ptr(out), n), "add")


BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}
UNARY_OPS = {"relu": 0, "sigmoid": 1, "silu": 2, "gelu_tanh": 3, "gelu": 4, "erf": 5, "tanh": 6}
MODE_FULL, MODE_SCALAR, MODE_BIAS = 0, 1, 2


def binary_dev(op: str, a, b, out, n: int, a_mode: int = MODE_FULL, b_mode: int = MODE_FULL, inner: int = 1) -> None:
    """out[i] = a[ia] op b[ib] on device operands (skainet_f32_binary's contract: full / scalar / bias operand modes)."""
    check(_lib.hip().skainet_hip_f32_binary_dev(BINARY_OPS[op], _ptr(a), a_mode, _ptr(b), b_mode, _ptr(out), n, inner), "binary")


def unary_dev(op: str, x, out, n: int) -> None:
    check(_lib.hip().skainet_hip_f32_unary_dev(UNARY_OPS[op], _ptr(x), _ptr(out), n), "unary")


def reduce_all_dev(x, n: int, out, mean: bool = False) -> None:
    check(_lib.hip().skainet_hip_f32_reduce_all_dev(_ptr(x), n, int(mean), _ptr(out)), "reduce_all")


def reduce_axis_dev(x, outer: int, red: int, inner: int, out, mean: bool = False) -> None:
    check(_lib.hip().skainet_hip_f32_reduce_axis_dev(_ptr(x), outer, red, inner, int(mean), _ptr(out)), "reduce_axis")


def argmax_rows_dev(x, rows: int, cols: int, out) -> None:
    check(_lib.hip().skainet_hip_f32_argmax_rows_dev(_ptr(x), rows, cols, _ptr(out)), "argmax_rows")


def argmax_rows_noalloc_dev(x, rows: int, cols: int, out) -> None:
    """argmax_rows_dev without any device allocation: scratch is a fixed array inside the library, at most 64 rows."""
    check(_lib.hip().skainet_hip_f32_argmax_rows_noalloc_dev(_ptr(x), rows, cols, _ptr(out)), "argmax_rows_noalloc")


def rope_scatter_dev(x, out, tokens, heads, head_dim, pos_start=0, pos_dev=None, theta=10000.0, rotate=True,
                     out_head_stride=None, out_row_is_pos=False, in_row_pitch=None) -> None:
    if out_head_stride is None:
        out_head_stride = tokens * head_dim
    if in_row_pitch is None:
        in_row_pitch = heads * head_dim
    check(_lib.hip().skainet_hip_f32_rope_scatter_dev(_ptr(x), in_row_pitch, _ptr(out), tokens, heads, head_dim, pos_start,
                                                      _ptr(pos_dev), theta, int(rotate), out_head_stride, int(out_row_is_pos)),
          "rope_scatter")


def swiglu_pairs_dev(gate_up, out, n: int) -> None:
    """out[i] = silu(gate_up[2i]) * gate_up[2i + 1] for i < n."""
    check(_lib.hip().skainet_hip_f32_swiglu_pairs_dev(_ptr(gate_up), _ptr(out), n), "swiglu_pairs")


def rope_qkv_dev(qkv, q_out, k_cache, v_cache, tokens, heads, kv_heads, head_dim, kv_capacity, pos_start=0, pos_dev=None,
                 theta=10000.0) -> None:
    check(_lib.hip().skainet_hip_f32_rope_qkv_dev(_ptr(qkv), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), tokens, heads, kv_heads,
                                                  head_dim, kv_capacity, pos_start, _ptr(pos_dev), theta), "rope_qkv")


def heads_to_rows_dev(x, out, heads, tokens, head_dim) -> None:
    check(_lib.hip().skainet_hip_f32_heads_to_rows_dev(_ptr(x), _ptr(out), heads, tokens, head_dim), "heads_to_rows")


def i32_increment_dev(value, delta: int) -> None:
    check(_lib.hip().skainet_hip_i32_increment_dev(_ptr(value), delta), "i32_increment")


def rope_table_dev(pos_dev, theta: float, head_dim: int, table) -> None:
    """table[2i], table[2i + 1] = cos, sin of (*pos_dev) * theta^(-2i / head_dim)."""
    check(_lib.hip().skainet_hip_f32_rope_table_dev(_ptr(pos_dev), theta, head_dim, _ptr(table)), "rope_table")


def decode_advance_dev(pos, kv_len, token, log, capacity: int) -> None:
    """*pos += 1, *kv_len += 1, log[*pos] = *token on the device; nothing changes once *pos == capacity."""
    check(_lib.hip().skainet_hip_decode_advance_dev(_ptr(pos), _ptr(kv_len), _ptr(token), _ptr(log), capacity), "decode_advance")


def i32_store_at_dev(dst, index_dev, offset: int, src) -> None:
    check(_lib.hip().skainet_hip_i32_store_at_dev(_ptr(dst), _ptr(index_dev), offset, _ptr(src)), "i32_store_at")


class Graph:
    """Records the device entries issued inside the `with` block into a HIP graph; `launch()` replays them."""

    def __init__(self):
        self._g = 0

    def __enter__(self):
        check(_lib.hip().skainet_hip_graph_begin(), "graph_begin")
        return self

    def __exit__(self, exc_type, exc, tb):
        g = _lib.hip().skainet_hip_graph_end()
        if not g and exc_type is None:
            raise HipError("graph_end: " + _lib.last_error())
        self._g = g or 0
        return False

    def launch(self) -> None:
        check(_lib.hip().skainet_hip_graph_launch(self._g), "graph_launch")

    def valid(self) -> bool:
        """False once the library reallocated this thread's scratch after the recording: launch() would be refused."""
        return bool(self._g) and bool(_lib.hip().skainet_hip_graph_valid(self._g))

    def sync(self) -> None:
        check(_lib.hip().skainet_hip_graph_sync(self._g), "graph_sync")

    def close(self) -> None:
        if self._g:
            _lib.hip().skainet_hip_graph_free(self._g)
            self._g = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def fp32_matmul_dev(a, a_offset, a_stride, b, b_offset, b_stride, out, out_offset, out_stride, m, n, k) -> None:
    check(_lib.hip().skainet_hip_fp32_matmul_dev(_ptr(a), a_offset, a_stride, _ptr(b), b_offset, b_stride, _ptr(out),
                                                 out_offset, out_stride, m, n, k), "fp32_matmul")


def fp32_matmul_wt_dev(x, x_offset, w, w_offset, out, out_offset, m, n, k) -> None:
    check(_lib.hip().skainet_hip_fp32_matmul_wt_dev(_ptr(x), x_offset, _ptr(w), w_offset, _ptr(out), out_offset, m, n, k),
          "fp32_matmul_wt")


class Timer:
    """HIP-event stopwatch on the calling thread's launch stream."""

    def __enter__(self):
        check(_lib.hip().skainet_hip_timer_begin(), "timer_begin")
        self.ms = None
        return self

    def __exit__(self, *exc):
        ms = _lib.hip().skainet_hip_timer_end_ms()
        if ms < 0:
            raise HipError("timer_end: " + _lib.last_error())
        self.ms = ms
        return False


# ---------------------------------------------------------------------------------------------- SPI kernels (host arrays)

def _raise_if_failed(what: str) -> None:
    # The void host entries clear the thread's error text on entry; a message afterwards means this call failed.
    now = _lib.hip().skainet_hip_last_error()
    if now:
        raise HipError(f"{what}: {now.decode('utf-8', 'replace')}")


class HipPackedMatmulKernel:
    """Q4KMatmulKernel / Q6KMatmulKernel / Q8_0MatmulKernel (and the Q4_0 / Q5_0 / Q5_1 / Q5_K ones): one activation row
    times an input-block-major weight."""

    def __init__(self, encoding: str):
        self.encoding = encoding
        self._id, self.block_size, self.bytes_per_block = ENCODINGS[encoding]
        short = {"Q4_K": "q4k", "Q6_K": "q6k", "Q8_0": "q8_0", "Q4_0": "q4_0", "Q5_0": "q5_0", "Q5_1": "q5_1", "Q5_K": "q5k"}[encoding]
        self._fn_name, self._fn_rm_name = f"skainet_hip_{short}_matmul", f"skainet_hip_{short}_matmul_rm"

    def _run(self, fn_name, input, input_offset, weight, weight_byte_offset, input_dim, output_dim, output, output_offset):
        if input_dim % self.block_size != 0:
            raise ValueError(f"Hip{self.encoding}MatmulKernel: inputDim must be a multiple of {self.block_size}; got {input_dim}")
        _require_available()
        _f32(input, "input"); _f32(output, "output")
        if weight.dtype != np.uint8:
            raise TypeError("weight must be a uint8 numpy array")
        need = weight_byte_offset + output_dim * (input_dim // self.block_size) * self.bytes_per_block
        if weight.size < need or input.size < input_offset + input_dim or output.size < output_offset + output_dim:
            raise ValueError("operand shorter than the dimensions require")
        lib = _lib.hip()
        getattr(lib, fn_name)(input.ctypes.data, input_offset, weight.ctypes.data, weight_byte_offset, input_dim, output_dim,
                              output.ctypes.data, output_offset)
        _raise_if_failed(fn_name)

    def matmul(self, input, input_offset, weight, weight_byte_offset, input_dim, output_dim, output, output_offset):
        self._run(self._fn_name, input, input_offset, weight, weight_byte_offset, input_dim, output_dim, output, output_offset)

    def matmul_row_major(self, input, input_offset, weight, weight_byte_offset, input_dim, output_dim, output, output_offset):
        """Same product for a weight in canonical GGUF order (the `_rm` native entries)."""
        self._run(self._fn_rm_name, input, input_offset, weight, weight_byte_offset, input_dim, output_dim, output, output_offset)


class HipFp32MatmulKernel:
    def matmul(self, a, a_offset, a_stride, b, b_offset, b_stride, out, out_offset, out_stride, m, n, k):
        _require_available()
        lib = _lib.hip()
        lib.skainet_hip_fp32_matmul(_f32(a, "a").ctypes.data, a_offset, a_stride, _f32(b, "b").ctypes.data, b_offset, b_stride,
                                    _f32(out, "out").ctypes.data, out_offset, out_stride, m, n, k)
        _raise_if_failed("fp32_matmul")


class HipNarrowFloatMatmulKernel:
    """Bf16MatmulKernel / Fp16MatmulKernel (skainet-backend-api kernel/NarrowFloatMatmulKernel.kt:25-49,
    ScalarBf16MatmulKernel.kt:19-46): C(m, n) = A(m, k) B(k, n) with B two bytes per element (little-endian bf16 or IEEE
    binary16), byte offset and byte row stride for B, float strides for A and C, fp32 sums, k == 0 zeroes the block."""

    def __init__(self, codec: str):
        if codec not in ("BFloat16", "Float16"):
            raise ValueError(f"codec must be BFloat16 or Float16, got {codec!r}")
        self.codec = codec

    def matmul(self, a, a_offset, a_stride, b, b_byte_offset, b_byte_stride, out, out_offset, out_stride, m, n, k):
        if m < 0 or n < 0 or k < 0:
            raise ValueError(f"{self.codec} matmul: m, n, k must be non-negative; got m={m} n={n} k={k}")
        _require_available()
        lib = _lib.hip()
        if not (isinstance(b, np.ndarray) and b.dtype == np.uint8 and b.flags.c_contiguous):
            raise TypeError("b must be a C-contiguous uint8 numpy array")
        fn = lib.skainet_hip_bf16_matmul if self.codec == "BFloat16" else lib.skainet_hip_fp16_matmul
        fn(_f32(a, "a").ctypes.data, a_offset, a_stride, b.ctypes.data, b_byte_offset, b_byte_stride,
           _f32(out, "out").ctypes.data, out_offset, out_stride, m, n, k)
        _raise_if_failed(f"{self.codec} matmul")


class HipFp32MatmulWtKernel:
    def matmul_wt(self, input, input_offset, weight, weight_offset, out, out_offset, m, n, k):
        _require_available()
        lib = _lib.hip()
        lib.skainet_hip_fp32_matmul_wt(_f32(input, "input").ctypes.data, input_offset, _f32(weight, "weight").ctypes.data,
                                       weight_offset, _f32(out, "out").ctypes.data, out_offset, m, n, k)
        _raise_if_failed("fp32_matmul_wt")


class HipFp32SoftmaxKernel:
    def softmax_rows(self, input, input_offset, out, out_offset, rows, cols, log):
        _require_available()
        lib = _lib.hip()
        lib.skainet_hip_f32_softmax_rows(_f32(input, "input").ctypes.data + 4 * input_offset,
                                         _f32(out, "out").ctypes.data + 4 * out_offset, rows, cols, int(log))
        _raise_if_failed("softmax_rows")


class HipFp32NormKernel:
    def layer_norm(self, input, input_offset, gamma, beta, out, out_offset, rows, cols, eps):
        _require_available()
        lib = _lib.hip()
        lib.skainet_hip_f32_layer_norm(_f32(input, "input").ctypes.data + 4 * input_offset, _ptr(gamma), _ptr(beta),
                                       _f32(out, "out").ctypes.data + 4 * out_offset, rows, cols, eps)
        _raise_if_failed("layer_norm")

    def rms_norm(self, input, input_offset, gamma, out, out_offset, rows, cols, eps):
        _require_available()
        lib = _lib.hip()
        lib.skainet_hip_f32_rms_norm(_f32(input, "input").ctypes.data + 4 * input_offset, _ptr(gamma),
                                     _f32(out, "out").ctypes.data + 4 * out_offset, rows, cols, eps)
        _raise_if_failed("rms_norm")


class HipFp32AttentionKernel:
    def sdpa(self, query, key, value, out, batch, heads, kv_heads, seq_q, seq_kv, head_dim, scale, causal, window,
             right_context, key_lengths=None, mask=None, mask_dims=None):
        """Fp32AttentionKernel.sdpa: whole contiguous arrays, `scale` applied as given, `out` fully overwritten."""
        if window < 0 or right_context < 0 or (right_context != 0 and window == 0):
            raise ValueError("SDPA: window/rightContext out of contract")   # AttentionMask.validate
        _require_available()
        md = [0, 0, 0, 0]
        if mask is not None:
            dims = list(mask_dims) if mask_dims is not None else list(mask.shape)
            md = [1] * (4 - len(dims)) + dims
        kl = None if key_lengths is None else np.ascontiguousarray(key_lengths, dtype=np.int32)
        lib = _lib.hip()
        lib.skainet_hip_f32_sdpa(_f32(query, "query").ctypes.data, _f32(key, "key").ctypes.data, _f32(value, "value").ctypes.data,
                                 _f32(out, "out").ctypes.data, batch, heads, kv_heads, seq_q, seq_kv, head_dim, scale,
                                 int(causal), window, right_context, _ptr(kl), _ptr(mask), *md)
        _raise_if_failed("sdpa")


class HipRowMajorMatmulKernel:
    """The ViewKernel for matmul(F32 dense contiguous x F32/<enc> BLOCKED_ROW_MAJOR): a [rows, k] activation against a
    GGUF-ordered [n, k] weight, all rows in one call. The weight is uploaded on first use and cached by the identity
    of its byte array, like the reference's resident-weight caches
    (/root/reference/skainet-backends/skainet-backend-wasm-simd/src/wasmJsMain/kotlin/sk/ainet/exec/wasm/WasmKernels.kt:206-223)."""

    CACHE_LIMIT = 256

    def __init__(self, encoding: str):
        self.encoding = encoding
        self.name = f"hip-{encoding}-rm"
        self._cache: dict = {}
        self._lock = threading.Lock()

    def _resident(self, weight: np.ndarray, n: int, k: int) -> DeviceWeight:
        key = (weight.ctypes.data, weight.size, n, k)
        with self._lock:
            hit = self._cache.get(key)
            if hit is not None:
                return hit[0]
            w = DeviceWeight.upload(self.encoding, weight, n, k)
            if len(self._cache) >= self.CACHE_LIMIT:
                self._cache.pop(next(iter(self._cache)))   # evict the oldest
            self._cache[key] = (w, weight)                  # hold the array so its address stays unique
            return w

    def run(self, a: np.ndarray, w: np.ndarray, n: int, out: np.ndarray) -> None:
        """One call of the library's host-array entry: the activation rows go up, the product comes down, the weight
        stays where it is. Nothing is allocated per call."""
        _require_available()
        rows, k = a.shape
        self._resident(w, n, k).matmul_host(a, out)


class HipKernelProvider:
    """KernelProvider for the HIP backend: outranks scalar (0), Panama (50) and native (100)."""

    name = "hip"
    priority = PRIORITY_HIP

    def is_available(self) -> bool:
        return is_available()

    def matmul_fp32(self): return HipFp32MatmulKernel() if is_available() else None
    def matmul_fp32_wt(self): return HipFp32MatmulWtKernel() if is_available() else None
    def matmul_bf16(self): return HipNarrowFloatMatmulKernel("BFloat16") if is_available() else None
    def matmul_fp16(self): return HipNarrowFloatMatmulKernel("Float16") if is_available() else None
    def matmul_q4k(self): return HipPackedMatmulKernel("Q4_K") if is_available() else None
    def matmul_q6k(self): return HipPackedMatmulKernel("Q6_K") if is_available() else None
    def matmul_q8_0(self): return HipPackedMatmulKernel("Q8_0") if is_available() else None
    def matmul_q4_0(self): return HipPackedMatmulKernel("Q4_0") if is_available() else None
    def matmul_q5_0(self): return HipPackedMatmulKernel("Q5_0") if is_available() else None
    def matmul_q5_1(self): return HipPackedMatmulKernel("Q5_1") if is_available() else None
    def matmul_q5k(self): return HipPackedMatmulKernel("Q5_K") if is_available() else None
    def softmax_fp32(self): return HipFp32SoftmaxKernel() if is_available() else None
    def norm_fp32(self): return HipFp32NormKernel() if is_available() else None
    def attention_fp32(self): return HipFp32AttentionKernel() if is_available() else None

    def supports(self, op_name: str, dtype_keys) -> bool:
        """KernelProvider.supports (KernelProvider.kt:161-190): true iff the accessor for the combination returns a kernel.
        One key ["Float32"]: "softmax", "layer_norm", "rms_norm", "sdpa"; two keys [input, weight]: "matmul" over the
        weight names below, "matmul_wt" over Float32 x Float32."""
        if not is_available():
            return False
        keys = list(dtype_keys)
        if len(keys) == 1:
            return keys[0] == "Float32" and op_name in ("softmax", "layer_norm", "rms_norm", "sdpa")
        if len(keys) != 2 or keys[0] != "Float32":
            return False
        if op_name == "matmul_wt":
            return keys[1] == "Float32"
        return op_name == "matmul" and keys[1] in ("Float32", "BFloat16", "Float16", "Q4_K", "Q6_K", "Q8_0", "Q4_0", "Q5_0",
                                                   "Q5_1", "Q5_K")
