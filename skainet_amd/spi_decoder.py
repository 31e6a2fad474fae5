"""Greedy decode through the kernel SPI alone: every operand that crosses the library boundary is a host array.

This is what a decoder gets when it is written against the unchanged kernel interfaces of the reference
(/root/reference/skainet-backends/skainet-backend-api/src/commonMain/kotlin/sk/ainet/backend/api/kernel/MatmulKernels.kt:11-40
ViewKernel.run, Fp32NormKernel.kt:31-79, Fp32AttentionKernel.kt:18-51) and picks this backend up through the provider
registry: weights stay resident on the device (the identity cache of HipRowMajorMatmulKernel), but the hidden state, the
KV cache and every intermediate row live on the host, so each linear is an upload, a launch, a download and a wait, and
attention stages the keys and values of the layer on every call. LlamaDecoder keeps all of that on the device instead;
this class exists so the two routes can be measured side by side and so the host route stays tested end to end.

Row ops the SPI has no kernel interface for (RoPE, SwiGLU, the residual adds, arg-max) run in numpy on the host, as the
reference's CPU ops would."""
from __future__ import annotations

import time
from typing import List

import numpy as np

from . import kernels
from .decoder import DeviceBuffer, LlamaWeights


class SpiDecoder:
    def __init__(self, weights: LlamaWeights):
        c = self.cfg = weights.cfg
        self.w = weights
        self.norm_kernel = kernels.HipFp32NormKernel()
        self.attn_kernel = kernels.HipFp32AttentionKernel()
        # norm gains as host arrays, the SPI's operand type
        self.attn_gain = [L.attn_norm.download(np.float32, c.hidden) for L in weights.layers]
        self.ffn_gain = [L.ffn_norm.download(np.float32, c.hidden) for L in weights.layers]
        self.out_gain = weights.out_norm.download(np.float32, c.hidden)
        self.k_cache = np.zeros((c.layers, c.kv_heads, c.ctx_max, c.head_dim), np.float32)
        self.v_cache = np.zeros((c.layers, c.kv_heads, c.ctx_max, c.head_dim), np.float32)
        self.pos = 0
        self.token = 0
        self.logits = np.zeros((1, c.vocab), np.float32)
        half = c.head_dim // 2
        # the device kernels' expression, evaluated in fp32
        self._freq = np.power(np.float32(c.rope_theta), np.float32(-2.0) * np.arange(half, dtype=np.float32) / np.float32(c.head_dim))
        self._ids = DeviceBuffer(4)
        self._row = DeviceBuffer(4 * c.hidden)
        self.calls = 0                 # library calls that cross the boundary with host operands
        self.matmul_seconds = 0.0      # wall time inside the host-array product calls
        self.matmul_calls = 0
        self.attention_seconds = 0.0   # wall time inside the attention calls (they stage the layer's keys and values)

    # ------------------------------------------------------------------ host-side row ops
    def _rope(self, x: np.ndarray, heads: int, pos: int) -> np.ndarray:
        """Adjacent pairs (x[2i], x[2i+1]) of every head rotated by pos * theta^(-2i / head_dim)."""
        c = self.cfg
        ang = (np.float32(pos) * self._freq).astype(np.float32)
        cs, sn = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
        p = x.reshape(heads, c.head_dim // 2, 2)
        out = np.empty_like(p)
        out[..., 0] = p[..., 0] * cs - p[..., 1] * sn
        out[..., 1] = p[..., 0] * sn + p[..., 1] * cs
        return out.reshape(heads, c.head_dim)

    def _linear(self, w: kernels.DeviceWeight, a: np.ndarray, out: np.ndarray) -> None:
        t0 = time.perf_counter()
        w.matmul_host(a, out)
        self.matmul_seconds += time.perf_counter() - t0
        self.matmul_calls += 1
        self.calls += 1

    def _embed(self, token: int) -> np.ndarray:
        c = self.cfg
        self._ids.upload(np.array([token], np.int32))
        self.w.tok_embd.dequantize_rows(self._ids, 1, self._row)
        kernels.sync()
        self.calls += 1
        return self._row.download(np.float32, c.hidden).reshape(1, c.hidden)

    # ------------------------------------------------------------------ one token
    def step(self, token: int) -> int:
        """Feed `token` at the current position, return the greedy next token."""
        c = self.cfg
        if not 0 <= token < c.vocab:
            raise ValueError(f"token id {token} is outside the vocabulary [0, {c.vocab})")
        if self.pos >= c.ctx_max:
            raise ValueError(f"position {self.pos} is past the context limit {c.ctx_max}")
        h = self._embed(token)
        normed = np.empty_like(h)
        qkv = np.empty((1, c.q_dim + 2 * c.kv_dim), np.float32)
        attn = np.empty((1, c.heads, 1, c.head_dim), np.float32)
        proj = np.empty((1, c.hidden), np.float32)
        gate_up = np.empty((1, 2 * c.ffn), np.float32)
        scale = float(1.0 / np.sqrt(c.head_dim))
        n_kv = self.pos + 1
        for li, L in enumerate(self.w.layers):
            self.norm_kernel.rms_norm(h, 0, self.attn_gain[li], normed, 0, 1, c.hidden, c.rms_eps)
            self._linear(L.wqkv, normed, qkv)
            q = self._rope(qkv[0, :c.q_dim], c.heads, self.pos)
            k = self._rope(qkv[0, c.q_dim:c.q_dim + c.kv_dim], c.kv_heads, self.pos)
            self.k_cache[li, :, self.pos] = k
            self.v_cache[li, :, self.pos] = qkv[0, c.q_dim + c.kv_dim:].reshape(c.kv_heads, c.head_dim)
            keys = np.ascontiguousarray(self.k_cache[li, :, :n_kv])[None]
            values = np.ascontiguousarray(self.v_cache[li, :, :n_kv])[None]
            t0 = time.perf_counter()
            self.attn_kernel.sdpa(np.ascontiguousarray(q.reshape(1, c.heads, 1, c.head_dim)), keys, values, attn,
                                  1, c.heads, c.kv_heads, 1, n_kv, c.head_dim, scale, True, 0, 0)
            self.attention_seconds += time.perf_counter() - t0
            self._linear(L.wo, attn.reshape(1, c.q_dim), proj)
            h = h + proj
            self.norm_kernel.rms_norm(h, 0, self.ffn_gain[li], normed, 0, 1, c.hidden, c.rms_eps)
            self._linear(L.w_gate_up, normed, gate_up)
            g, u = gate_up[0, 0::2], gate_up[0, 1::2]              # row 2j = gate row j, row 2j + 1 = up row j
            act = np.ascontiguousarray((g / (np.float32(1.0) + np.exp(-g)) * u).reshape(1, c.ffn), dtype=np.float32)
            self._linear(L.w_down, act, proj)
            h = h + proj
            self.calls += 3        # two norms and the attention
        self.norm_kernel.rms_norm(h, 0, self.out_gain, normed, 0, 1, c.hidden, c.rms_eps)
        self._linear(self.w.head, normed, self.logits)
        self.calls += 1
        self.pos += 1
        self.token = int(np.argmax(self.logits[0]))
        return self.token

    def prefill(self, token_ids) -> int:
        """Token by token: the SPI's attention takes one query block against whole arrays, and this route is about its
        per-call cost, not about prompt throughput."""
        nxt = 0
        for t in np.asarray(token_ids, dtype=np.int64).reshape(-1):
            nxt = self.step(int(t))
        return nxt

    def decode(self, steps: int) -> List[int]:
        out = []
        for _ in range(steps):
            out.append(self.step(self.token))
        return out

    def close(self) -> None:
        self._ids.close()
        self._row.close()
