"""The resident-activation ops class of the HIP backend: the host-side mirror of a `HipOps : DefaultCpuOpsBase`.

The reference keeps activations resident across ops in exactly one tier, the browser's
(/root/reference/skainet-backends/skainet-backend-wasm-simd/src/wasmJsMain/kotlin/sk/ainet/exec/wasm/WasmCpuOps.kt:47-56):
a `TensorOps` whose dense matmuls (:180-236), elementwise arithmetic (:240-277), activations (:281-312), reductions
(:316-348), softmax (:352-374), fused norms (:383-420) and scaled-dot-product attention (:428) run in the sidecar and
leave their outputs in the sidecar's memory (`WasmLinearStorage.kt:34`), so that a chain of ops never copies an activation
back to the heap. This module is that class for the GPU: the same method set, every output a `HipTensor` whose bytes
live in device memory (the `HipDeviceStorage` of the Kotlin module), every method one device entry of
include/skainet_hip.h. A packed weight reaches `matmul_weight_transposed` as a `kernels.DeviceWeight` (what
`KernelDispatch` hands a view kernel, MatmulKernels.kt:11-40); a dense one as a `HipTensor`.

Outputs come from a `ForwardScope` (Scope.kt:108: a per-step slab with `reset()`), so a step that allocates the same
sequence of outputs gets the same addresses every time -- which is what lets a whole decode step built from these
generic ops be recorded into a HIP graph. Without a scope an output owns a device allocation of its own.

Beyond the reference's TensorOps set (the reference has no transformer; RoPE, the KV cache and the sampler live in an
external repository) the class carries the four glue ops a decoder needs, marked as such below: `embedding_rows`,
`rope_scatter`, `heads_to_rows` and `argmax_rows`.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple, Union

import numpy as np

from . import _lib, kernels
from ._lib import HipError, check


class _Allocation:
    """Device bytes from skainet_hip_malloc, freed with the object."""

    def __init__(self, nbytes: int):
        self.nbytes = max(int(nbytes), 1)
        self.ptr = _lib.hip().skainet_hip_malloc(self.nbytes)
        if not self.ptr:
            raise HipError("malloc: " + _lib.last_error())

    def close(self) -> None:
        if self.ptr:
            _lib.hip().skainet_hip_free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class ForwardScope:
    """A slab of device memory handed out front to back; `reset()` makes the whole slab free again (Scope.kt:108-215:
    per-step activations belong to a forward scope, freed together). Allocations are 256-byte aligned."""

    def __init__(self, capacity_bytes: int):
        kernels._require_available()
        self._slab = _Allocation(capacity_bytes)
        self.capacity = int(capacity_bytes)
        self._top = 0
        self.high_water = 0
        self.generation = 0          # resets so far: a tensor handed out before the last one is stale (Scope.kt:206-215)

    def allocate(self, nbytes: int) -> int:
        at = (self._top + 255) & ~255
        if at + nbytes > self.capacity:
            raise HipError(f"forward scope of {self.capacity} bytes is full ({at} in use, {nbytes} asked)")
        self._top = at + int(nbytes)
        self.high_water = max(self.high_water, self._top)
        return self._slab.ptr + at

    def reset(self) -> None:
        """End of a step: every tensor handed out so far is invalid (its next use raises), the slab starts over."""
        self._top = 0
        self.generation += 1

    def close(self) -> None:
        self.generation += 1
        self._slab.close()


class HipTensor:
    """A dense tensor whose bytes are resident on the device (fp32 unless `dtype` says int32). `owner` keeps the
    allocation alive: an `_Allocation`, a `ForwardScope`, or another tensor (views)."""

    __slots__ = ("shape", "_ptr", "owner", "dtype", "_scope", "_generation")

    def __init__(self, shape: Sequence[int], ptr: int, owner, dtype=np.float32):
        self.shape = tuple(int(s) for s in shape)
        self._ptr = int(ptr)
        self.owner = owner
        self.dtype = np.dtype(dtype)
        # a tensor of a forward scope (or a view of one) lives until that scope's next reset
        self._scope = owner if isinstance(owner, ForwardScope) else getattr(owner, "_scope", None)
        self._generation = owner.generation if isinstance(owner, ForwardScope) else getattr(owner, "_generation", 0)

    @property
    def ptr(self) -> int:
        """The device address; raises once the forward scope that handed the bytes out has been reset or closed (the
        reference closes a scope's storages at reset, so a later use throws: Scope.kt:206-215)."""
        if self._scope is not None and self._scope.generation != self._generation:
            raise HipError(f"tensor {self.shape} belongs to a forward scope that has been reset since")
        return self._ptr

    @property
    def volume(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n

    @property
    def nbytes(self) -> int:
        return self.volume * self.dtype.itemsize

    def data_ptr(self) -> int:
        return self.ptr

    def reshape(self, *shape: int) -> "HipTensor":
        t = HipTensor(shape, self.ptr, self, self.dtype)
        if t.volume != self.volume:
            raise ValueError(f"reshape of {self.shape} to {tuple(shape)}")
        return t

    def rows(self, start: int, count: int) -> "HipTensor":
        """A view of `count` leading-dimension slices from `start` (contiguous: no copy)."""
        if start < 0 or count < 0 or start + count > self.shape[0]:
            raise ValueError(f"rows [{start}, {start + count}) of {self.shape}")
        inner = self.volume // max(self.shape[0], 1)
        return HipTensor((count,) + self.shape[1:], self.ptr + start * inner * self.dtype.itemsize, self, self.dtype)

    def numpy(self) -> np.ndarray:
        """The heap mirror: one synchronous download."""
        out = np.empty(self.shape, dtype=self.dtype)
        if out.size:
            check(_lib.hip().skainet_hip_sync(), "sync")
            check(_lib.hip().skainet_hip_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes), "d2h")
        return out


Weight = Union[HipTensor, "kernels.DeviceWeight"]


def _broadcast_shape(a: Tuple[int, ...], b: Tuple[int, ...]) -> Tuple[int, ...]:
    return tuple(np.broadcast_shapes(a, b))


class HipOps:
    """Device-resident tensor ops. Shape errors raise ValueError before any device work (IllegalArgumentException in the
    Kotlin class), device failures HipError (IllegalStateException); there is no CPU path behind any of them."""

    def __init__(self, scope: Optional[ForwardScope] = None):
        kernels._require_available()
        self.scope = scope
        self._lib = _lib.hip()

    # ---- operands and outputs -----------------------------------------------------------------------------------------
    @staticmethod
    def _live(*tensors) -> None:
        """Operands are checked before an output is taken from the scope: a stale one raises without costing slab bytes."""
        for t in tensors:
            if isinstance(t, HipTensor):
                t.ptr

    def _out(self, shape: Sequence[int], dtype=np.float32) -> HipTensor:
        n = int(np.prod(shape, dtype=np.int64)) * np.dtype(dtype).itemsize
        if self.scope is not None:
            return HipTensor(shape, self.scope.allocate(n), self.scope, dtype)
        a = _Allocation(n)
        return HipTensor(shape, a.ptr, a, dtype)

    def to_resident(self, array: np.ndarray) -> HipTensor:
        """Upload once (WasmCpuOps.kt:154 toResident): an input that many ops will read."""
        a = np.ascontiguousarray(array)
        if a.dtype not in (np.float32, np.int32):
            a = a.astype(np.float32)
        t = self._out(a.shape, a.dtype)
        if a.size:
            check(self._lib.skainet_hip_memcpy_h2d(t.ptr, a.ctypes.data, a.nbytes), "h2d")
        return t

    def empty(self, shape: Sequence[int], dtype=np.float32) -> HipTensor:
        return self._out(shape, dtype)

    # ---- matmuls (WasmCpuOps.kt:180-236) -----------------------------------------------------------------------------
    def matmul(self, a: HipTensor, b: HipTensor) -> HipTensor:
        """Dense A(m, k) . B(k, n)."""
        if len(a.shape) != 2 or len(b.shape) != 2 or a.shape[1] != b.shape[0]:
            raise ValueError(f"Matrix multiplication shape mismatch: {a.shape} vs {b.shape}")
        m, k = a.shape
        n = b.shape[1]
        self._live(a, b)
        out = self._out((m, n))
        if m and n:
            check(self._lib.skainet_hip_fp32_matmul_dev(a.ptr, 0, k, b.ptr, 0, n, out.ptr, 0, n, m, n, k), "matmul")
        return out

    def matmul_weight_transposed(self, x: HipTensor, weight: Weight) -> HipTensor:
        """x(..., k) . W(n, k)^T. A dense weight is a HipTensor; a packed one (Q4_K, Q6_K, Q8_0, ...) a DeviceWeight, which
        takes the product its view kernel runs: GEMV kernels up to 8 rows, the MFMA dequant-GEMM above."""
        if isinstance(weight, HipTensor):
            if len(weight.shape) != 2:
                raise ValueError(f"weight must be [n, k]; got {weight.shape}")
            n, k = weight.shape
        else:
            n, k = weight.rows, weight.cols
        if not x.shape or x.shape[-1] != k:
            raise ValueError(f"matmulWeightTransposed shape mismatch: {x.shape} vs weight [{n}, {k}]")
        m = x.volume // k if k else 0
        self._live(x, weight)
        out = self._out(x.shape[:-1] + (n,))
        if m and n:
            if isinstance(weight, HipTensor):
                check(self._lib.skainet_hip_fp32_matmul_wt_dev(x.ptr, 0, weight.ptr, 0, out.ptr, 0, m, n, k), "matmul_wt")
            else:
                check(self._lib.skainet_hip_matmul_dev(weight._h, x.ptr, m, out.ptr), "matmul")
        return out

    # ---- elementwise (WasmCpuOps.kt:240-277) -------------------------------------------------------------------------
    @staticmethod
    def _mode(s: Tuple[int, ...], out: Tuple[int, ...]) -> int:
        """The operand's index mode against the broadcast output shape (WasmCpuOps.kt:232-238)."""
        if s == out:
            return kernels.MODE_FULL
        if int(np.prod(s, dtype=np.int64)) == 1:
            return kernels.MODE_SCALAR
        if s and out and s[-1] == out[-1] and all(d == 1 for d in s[:-1]):
            return kernels.MODE_BIAS
        raise ValueError(f"broadcast of {s} to {out} is not one of full / scalar / last-dimension bias")

    def _binary(self, op: str, a: HipTensor, b: HipTensor) -> HipTensor:
        shape = _broadcast_shape(a.shape, b.shape)
        am, bm = self._mode(a.shape, shape), self._mode(b.shape, shape)
        self._live(a, b)
        out = self._out(shape)
        n = out.volume
        if n:
            kernels.binary_dev(op, a, b, out, n, am, bm, shape[-1] if shape else 1)
        return out

    def add(self, a, b): return self._binary("add", a, b)
    def subtract(self, a, b): return self._binary("sub", a, b)
    def multiply(self, a, b): return self._binary("mul", a, b)
    def divide(self, a, b): return self._binary("div", a, b)

    # ---- activations (WasmCpuOps.kt:281-312) -------------------------------------------------------------------------
    def _unary(self, op: str, t: HipTensor) -> HipTensor:
        self._live(t)
        out = self._out(t.shape)
        if t.volume:
            kernels.unary_dev(op, t, out, t.volume)
        return out

    def relu(self, t): return self._unary("relu", t)
    def sigmoid(self, t): return self._unary("sigmoid", t)
    def silu(self, t): return self._unary("silu", t)
    def gelu(self, t, approximate: bool = False): return self._unary("gelu_tanh" if approximate else "gelu", t)
    def erf(self, t): return self._unary("erf", t)
    def tanh(self, t): return self._unary("tanh", t)

    # ---- reductions (WasmCpuOps.kt:316-348) --------------------------------------------------------------------------
    def _reduce(self, t: HipTensor, dim: Optional[int], mean: bool) -> HipTensor:
        self._live(t)
        if dim is None:
            out = self._out(())
            kernels.reduce_all_dev(t, t.volume, out, mean)
            return out
        rank = len(t.shape)
        if not -rank <= dim < rank:
            raise ValueError(f"dimension {dim} out of range for {t.shape}")
        dim %= rank
        outer = int(np.prod(t.shape[:dim], dtype=np.int64))
        red = t.shape[dim]
        inner = int(np.prod(t.shape[dim + 1:], dtype=np.int64))
        out = self._out(t.shape[:dim] + t.shape[dim + 1:])
        if out.volume:
            kernels.reduce_axis_dev(t, outer, red, inner, out, mean)
        return out

    def sum(self, t, dim: Optional[int] = None): return self._reduce(t, dim, False)
    def mean(self, t, dim: Optional[int] = None): return self._reduce(t, dim, True)

    # ---- softmax (WasmCpuOps.kt:352-374) and the fused norms (:383-420) ----------------------------------------------
    def _softmax(self, t: HipTensor, dim: int, log: bool) -> HipTensor:
        rank = len(t.shape)
        if rank == 0 or dim % rank != rank - 1:
            raise ValueError("softmax runs over the last dimension")
        cols = t.shape[-1]
        self._live(t)
        out = self._out(t.shape)
        if t.volume:
            kernels.softmax_rows_dev(t, out, t.volume // cols, cols, log)
        return out

    def softmax(self, t, dim: int = -1): return self._softmax(t, dim, False)
    def log_softmax(self, t, dim: int = -1): return self._softmax(t, dim, True)

    def rms_norm(self, x: HipTensor, gamma: Optional[HipTensor], eps: float) -> HipTensor:
        if not x.shape:
            raise ValueError("a norm needs a last dimension to run over")
        cols = x.shape[-1]
        if gamma is not None and gamma.volume != cols:
            raise ValueError(f"gamma of {gamma.shape} against rows of {cols}")
        self._live(x, gamma)
        out = self._out(x.shape)
        if x.volume:
            kernels.rms_norm_dev(x, gamma, out, x.volume // cols, cols, eps)
        return out

    def layer_norm(self, x: HipTensor, gamma: Optional[HipTensor], beta: Optional[HipTensor], eps: float) -> HipTensor:
        if not x.shape:
            raise ValueError("a norm needs a last dimension to run over")
        cols = x.shape[-1]
        for name, p in (("gamma", gamma), ("beta", beta)):
            if p is not None and p.volume != cols:
                raise ValueError(f"{name} of {p.shape} against rows of {cols}")
        self._live(x, gamma, beta)
        out = self._out(x.shape)
        if x.volume:
            kernels.layer_norm_dev(x, gamma, beta, out, x.volume // cols, cols, eps)
        return out

    # ---- attention (WasmCpuOps.kt:428) -------------------------------------------------------------------------------
    def scaled_dot_product_attention(self, q: HipTensor, k: HipTensor, v: HipTensor, scale: Optional[float] = None,
                                     causal: bool = False, window: int = 0, key_lengths: Optional[HipTensor] = None,
                                     seq_kv: Optional[int] = None) -> HipTensor:
        """q [B, H, Sq, D], k / v [B, Hkv, Skv, D] (the layout KvCacheStore.readKeys / readValues return). With `seq_kv`
        below k's third dimension, k / v are caches of that capacity whose first `seq_kv` rows are keys; `key_lengths`
        ([B] int32, resident) cuts each sequence's keys further, on the device."""
        if len(q.shape) != 4 or len(k.shape) != 4 or k.shape != v.shape or q.shape[0] != k.shape[0] or q.shape[3] != k.shape[3]:
            raise ValueError(f"attention operands {q.shape}, {k.shape}, {v.shape}")
        b, h, sq, d = q.shape
        kvh, cap = k.shape[1], k.shape[2]
        if kvh < 1 or h % kvh:
            raise ValueError(f"{h} query heads over {kvh} KV heads")
        skv = cap if seq_kv is None else int(seq_kv)
        if skv < 0 or skv > cap:
            raise ValueError(f"{skv} keys in caches of {cap} rows")
        self._live(q, k, v, key_lengths)
        out = self._out(q.shape)
        if out.volume:
            kernels.sdpa_cache_dev(q, k, v, out, b, h, kvh, sq, skv, cap, d, float(scale if scale is not None else d ** -0.5),
                                   causal, window, 0, key_lengths)
        return out

    # ---- glue a decoder needs; no counterpart among the reference's TensorOps ----------------------------------------
    def embedding_rows(self, table: "kernels.DeviceWeight", ids: HipTensor) -> HipTensor:
        """Rows `ids` ([count] int32, resident) of a packed embedding table, decoded to fp32 (the decode is the
        reference's, bit for bit: Q4_KTensorData.kt:133 and its siblings)."""
        count = ids.volume
        self._live(ids)
        out = self._out((count, table.cols))
        check(self._lib.skainet_hip_dequantize_rows_dev(table._h, ids.ptr, count, out.ptr), "dequantize_rows")
        return out

    def rope_scatter(self, x: HipTensor, out: HipTensor, heads: int, head_dim: int, theta: float, pos_start: int = 0,
                     pos_dev: Optional[HipTensor] = None, rotate: bool = True, cache_rows: bool = False) -> None:
        """Rotate adjacent pairs of x [tokens, heads * head_dim] by their position and scatter them head-major: into
        out [heads, tokens, head_dim], or with `cache_rows` into rows `pos ..` of a cache [heads, capacity, head_dim]
        (`rotate=False`: a plain scatter, for V). The position is pos_start, or the resident counter pos_dev."""
        tokens = x.volume // (heads * head_dim)
        stride = out.shape[1] * head_dim if cache_rows else tokens * head_dim
        kernels.rope_scatter_dev(x, out, tokens, heads, head_dim, pos_start, pos_dev, theta, rotate, stride, cache_rows,
                                 heads * head_dim)

    def heads_to_rows(self, x: HipTensor) -> HipTensor:
        """[heads, tokens, head_dim] -> [tokens, heads * head_dim] (the reshape in front of the output projection)."""
        heads, tokens, hd = x.shape
        self._live(x)
        out = self._out((tokens, heads * hd))
        kernels.heads_to_rows_dev(x, out, heads, tokens, hd)
        return out

    def argmax_rows(self, t: HipTensor, out: Optional[HipTensor] = None) -> HipTensor:
        cols = t.shape[-1]
        rows = t.volume // cols
        self._live(t, out)
        if out is None:
            out = self._out((rows,), np.int32)
        kernels.argmax_rows_dev(t, rows, cols, out)
        return out
