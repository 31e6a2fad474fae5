"""A Llama-shaped decoder stack written against the generic resident-activation ops class only.

`decoder.LlamaDecoder` drives the stack through the library's fused entries (norm + product + RoPE + cache append in one
launch, attention + projection as a pair, ...). This one is what a model built with the NN DSL looks like to the backend
when its `TensorOps` is `ops.HipOps`: every layer is the plain sequence rmsNorm, matmulWeightTransposed x 3, RoPE,
scaledDotProductAttention, matmulWeightTransposed, add, rmsNorm, matmulWeightTransposed x 2, silu, multiply,
matmulWeightTransposed, add -- one device entry per op, every intermediate a device-resident tensor, nothing fused by
name. It exists to put a number on that route (between the fused decoder and the host-array SPI route) and to hold the
ops class to the decoder's float64 checker.

Weights are the fused decoder's, seen op by op: q / k / v are row ranges of the concatenated [q; k; v] weight (views,
no copy), gate and up are the interleaved gate/up weight taken apart once (a copy at load time).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import numpy as np

from . import _lib, kernels
from ._lib import check
from .decoder import DeviceBuffer, LlamaConfig, LlamaWeights
from .ops import ForwardScope, HipOps, HipTensor


@dataclass
class OpsLayerWeights:
    attn_norm: HipTensor
    wq: kernels.DeviceWeight
    wk: kernels.DeviceWeight
    wv: kernels.DeviceWeight
    wo: kernels.DeviceWeight
    ffn_norm: HipTensor
    w_gate: kernels.DeviceWeight
    w_up: kernels.DeviceWeight
    w_down: kernels.DeviceWeight


class OpsLlamaWeights:
    """The weights of a `LlamaWeights` as one tensor per op."""

    def __init__(self, fused: LlamaWeights):
        c = self.cfg = fused.cfg
        self._fused = fused                         # owns the device bytes the views point into
        _, bs, nb = kernels.ENCODINGS[c.linear_encoding]
        row_bytes = c.hidden // bs * nb
        enc = c.linear_encoding

        def gain(buf: DeviceBuffer) -> HipTensor:
            return HipTensor((c.hidden,), buf.ptr, buf)

        def rows_of(w: kernels.DeviceWeight, first: int, count: int) -> kernels.DeviceWeight:
            return kernels.DeviceWeight.wrap(enc, w.data_ptr + first * row_bytes, count, c.hidden)

        self.layers: List[OpsLayerWeights] = []
        self._owned: List[DeviceBuffer] = []
        for L in fused.layers:
            # gate / up rows alternate in the fused weight: taken apart once, through the host
            gu = np.empty(L.w_gate_up.nbytes, np.uint8)
            check(_lib.hip().skainet_hip_memcpy_d2h(gu.ctypes.data, L.w_gate_up.data_ptr, gu.nbytes), "d2h")
            gu = gu.reshape(2 * c.ffn, row_bytes)
            halves = []
            for part in (0, 1):
                buf = DeviceBuffer(c.ffn * row_bytes).upload(np.ascontiguousarray(gu[part::2]))
                self._owned.append(buf)
                halves.append(kernels.DeviceWeight.wrap(enc, buf.ptr, c.ffn, c.hidden))
            self.layers.append(OpsLayerWeights(
                attn_norm=gain(L.attn_norm),
                wq=rows_of(L.wqkv, 0, c.q_dim), wk=rows_of(L.wqkv, c.q_dim, c.kv_dim), wv=rows_of(L.wqkv, c.q_dim + c.kv_dim, c.kv_dim),
                wo=L.wo, ffn_norm=gain(L.ffn_norm), w_gate=halves[0], w_up=halves[1], w_down=L.w_down))
        self.tok_embd, self.head = fused.tok_embd, fused.head
        self.out_norm = gain(fused.out_norm)


class OpsLlamaDecoder:
    """Prefill + greedy decode for batch 1 through `HipOps` alone; KV cache, position and current token on the device."""

    KEY_BUCKET = 512

    def __init__(self, weights: OpsLlamaWeights, max_prefill: int = 512):
        c = self.cfg = weights.cfg
        self.w = weights
        self.max_rows = max(1, max_prefill)
        rows = self.max_rows
        # one layer's intermediates: 6 hidden-sized, 4 q-sized, 2 kv-sized, 4 ffn-sized tensors of `rows` rows (one more of
        # each for alignment slack), and at the end of a step a logits row; the two scopes alternate between layers (a
        # layer's output outlives the next reset of the other scope only)
        per_layer = 4 * rows * (7 * c.hidden + 5 * c.q_dim + 3 * c.kv_dim + 5 * c.ffn) + 8 * c.vocab + (1 << 16)
        self.scopes = [ForwardScope(per_layer), ForwardScope(per_layer)]
        self.ops = [HipOps(s) for s in self.scopes]
        own = HipOps()
        self.k_cache = [own.empty((1, c.kv_heads, c.ctx_max, c.head_dim)) for _ in range(c.layers)]
        self.v_cache = [own.empty((1, c.kv_heads, c.ctx_max, c.head_dim)) for _ in range(c.layers)]
        self.pos = own.to_resident(np.zeros(1, np.int32))
        self.kv_len = own.to_resident(np.zeros(1, np.int32))
        self.token = own.to_resident(np.zeros(1, np.int32))
        self.generated = own.to_resident(np.zeros(c.ctx_max + 1, np.int32))
        self.logits: Optional[HipTensor] = None
        self.prompt_len = 0
        self._host_pos = 0
        self._graph: Optional[kernels.Graph] = None
        self._graph_bound = 0

    def _layer(self, li: int, h: HipTensor, rows: int, pos_start: int, pos_dev, seq_kv: int, kv_len_dev) -> HipTensor:
        c, L = self.cfg, self.w.layers[li]
        self.scopes[li & 1].reset()
        o = self.ops[li & 1]
        n1 = o.rms_norm(h, L.attn_norm, c.rms_eps)
        q = o.matmul_weight_transposed(n1, L.wq)
        k = o.matmul_weight_transposed(n1, L.wk)
        v = o.matmul_weight_transposed(n1, L.wv)
        qh = o.empty((1, c.heads, rows, c.head_dim))
        o.rope_scatter(q, qh.reshape(c.heads, rows, c.head_dim), c.heads, c.head_dim, c.rope_theta, pos_start, pos_dev)
        kc, vc = self.k_cache[li], self.v_cache[li]
        kc3, vc3 = kc.reshape(c.kv_heads, c.ctx_max, c.head_dim), vc.reshape(c.kv_heads, c.ctx_max, c.head_dim)
        o.rope_scatter(k, kc3, c.kv_heads, c.head_dim, c.rope_theta, pos_start, pos_dev, cache_rows=True)
        o.rope_scatter(v, vc3, c.kv_heads, c.head_dim, c.rope_theta, pos_start, pos_dev, rotate=False, cache_rows=True)
        a = o.scaled_dot_product_attention(qh, kc, vc, causal=True, key_lengths=kv_len_dev, seq_kv=seq_kv)
        a_rows = o.heads_to_rows(a.reshape(c.heads, rows, c.head_dim)) if rows > 1 else a.reshape(1, c.q_dim)
        h = o.add(h, o.matmul_weight_transposed(a_rows, L.wo))
        n2 = o.rms_norm(h, L.ffn_norm, c.rms_eps)
        act = o.multiply(o.silu(o.matmul_weight_transposed(n2, L.w_gate)), o.matmul_weight_transposed(n2, L.w_up))
        return o.add(h, o.matmul_weight_transposed(act, L.w_down))

    def _forward(self, ids: HipTensor, rows: int, pos_start: int, pos_dev, seq_kv: int, kv_len_dev) -> None:
        c = self.cfg
        self.scopes[1].reset()
        h = self.ops[1].embedding_rows(self.w.tok_embd, ids)      # layer 0 resets scope 0 only
        for li in range(c.layers):
            h = self._layer(li, h, rows, pos_start, pos_dev, seq_kv, kv_len_dev)
        o = self.ops[c.layers & 1]
        self.scopes[c.layers & 1].reset()
        n = o.rms_norm(h.rows(rows - 1, 1), self.w.out_norm, c.rms_eps)
        self.logits = o.matmul_weight_transposed(n, self.w.head)
        o.argmax_rows(self.logits, out=self.token)

    def prefill(self, token_ids) -> int:
        c = self.cfg
        ids = np.ascontiguousarray(token_ids, dtype=np.int64).reshape(-1)
        rows = int(ids.size)
        if rows < 1 or rows > self.max_rows or rows > c.ctx_max:
            raise ValueError(f"prompt of {rows} tokens does not fit (max_prefill {self.max_rows}, ctx {c.ctx_max})")
        if ids.min() < 0 or ids.max() >= c.vocab:
            raise ValueError(f"token id outside the vocabulary [0, {c.vocab})")
        ids_dev = HipOps().to_resident(ids.astype(np.int32))
        self._forward(ids_dev, rows, 0, None, rows, None)
        kernels.sync()
        for t, val in ((self.pos, rows), (self.kv_len, rows + 1)):
            a = np.array([val], np.int32)
            check(_lib.hip().skainet_hip_memcpy_h2d(t.ptr, a.ctypes.data, 4), "h2d")
        self.prompt_len = self._host_pos = rows
        kernels.i32_store_at_dev(self.generated, self.pos, 0, self.token)
        kernels.sync()
        return int(self.token.numpy()[0])

    def _key_bound(self, keys: int) -> int:
        b = self.KEY_BUCKET
        return min(self.cfg.ctx_max, (keys + b - 1) // b * b)

    def _decode_step(self, bound: Optional[int] = None) -> None:
        if bound is None:
            bound = self._key_bound(self._host_pos + 1)
        self._forward(self.token, 1, 0, self.pos, bound, self.kv_len)
        kernels.decode_advance_dev(self.pos, self.kv_len, self.token, self.generated, self.cfg.ctx_max)

    def _graph_step(self) -> None:
        keys = self._host_pos + 1
        if self._graph is not None and (not self._graph.valid() or keys > self._graph_bound):
            self._graph.close()
            self._graph = None
        if self._graph is None:
            bound = self._key_bound(keys + 1)
            self._decode_step(bound)               # eager once: sizes the library's scratch
            kernels.sync()
            self._host_pos += 1
            if self._host_pos < self.cfg.ctx_max:
                with kernels.Graph() as g:         # the scopes hand out the same addresses every step
                    self._decode_step(bound)
                self._graph, self._graph_bound = g, bound
            return
        self._graph.launch()
        self._host_pos += 1

    def run_steps(self, steps: int, use_graph: bool = True) -> None:
        if self._host_pos + steps > self.cfg.ctx_max:
            raise ValueError(f"{steps} more tokens would pass the context limit {self.cfg.ctx_max}")
        for _ in range(steps):
            if use_graph:
                self._graph_step()
            else:
                self._decode_step()
                self._host_pos += 1

    def decode(self, steps: int, use_graph: bool = True) -> np.ndarray:
        out = np.empty(steps, np.int32)
        for i in range(steps):
            self.run_steps(1, use_graph)
            out[i] = int(self.token.numpy()[0])
        return out

    def decode_timed(self, steps: int) -> float:
        import time
        kernels.sync()
        t0 = time.perf_counter()
        self.run_steps(steps)
        kernels.sync()
        return time.perf_counter() - t0

    def last_logits(self) -> np.ndarray:
        return self.logits.numpy().reshape(-1)

    def position(self) -> int:
        return int(self.pos.numpy()[0])

    def launches_per_token(self) -> int:
        """Device entries one decode step issues: 17 per layer (7 products, 2 norms, 3 scatters, attention, 4 elementwise
        ops), the embedding row, final norm, head product, arg-max and the position update."""
        return 17 * self.cfg.layers + 5

    def close(self) -> None:
        if self._graph is not None:
            self._graph.close()
            self._graph = None
        for s in self.scopes:
            s.close()
