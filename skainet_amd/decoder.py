"""A Llama-shaped decoder stack driven entirely through the backend's SPI-level device entries.

The reference repository has no transformer (RoPE, the decoder block and the sampler live in the external
SKaiNET-transformers repo; the nearest in-repo thing is the synthetic DecodeHarness,
/root/reference/skainet-backends/skainet-backend-cpu/src/commonTest/kotlin/sk/ainet/exec/harness/DecodeHarness.kt:49).
This driver is what such a model does with the kernel SPI: every linear layer is a packed-weight matmul
(`DeviceWeight.matmul`: GEMV kernels for decode, the MFMA GEMM for prefill), attention is the fused SDPA kernel over a
device KV cache laid out `[kv_heads, positions, head_dim]` per layer (the layout KvCacheStore.readKeys/readValues
return, .../lang/tensor/storage/KvCacheStore.kt:125-149), RMSNorm / SiLU*up / residual add / arg-max are the
reference ops' device twins. Activations never leave the device; a decode step can be recorded once into a HIP
graph and replayed (the position lives in device memory).

Block (standard Llama-3):  h += Wo . attn(rope(Wq n1), rope(Wk n1), Wv n1),  n1 = rmsnorm(h) * g1
                           h += Wdown . (silu(Wgate n2) * (Wup n2)),        n2 = rmsnorm(h) * g2
                           logits = Whead . (rmsnorm(h) * g_out);  greedy = first arg-max.
q/k/v weights are stored concatenated along the output rows ([q; k; v]) and gate/up interleaved row by row
(gate row j, up row j, gate row j + 1, ...), so each group is one pass over the activations and the SwiGLU pairs
come out of the product side by side. The norms, the residual adds and SwiGLU ride inside the products
(`DeviceWeight.matmul_fused`): a decode step is five launches per block (q/k/v product with norm, RoPE
and cache append; attention and its split merge; o product with residual; gate/up product with norm and SwiGLU; down
product with residual).
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import List, Optional

import numpy as np

from . import _lib, kernels
from ._lib import HipError, check


@dataclass
class LlamaConfig:
    layers: int = 32
    hidden: int = 4096
    heads: int = 32
    kv_heads: int = 8
    head_dim: int = 128
    ffn: int = 14336
    vocab: int = 128256
    rms_eps: float = 1e-5
    rope_theta: float = 500000.0
    ctx_max: int = 2048
    linear_encoding: str = "Q4_K"
    head_encoding: str = "Q6_K"

    @property
    def q_dim(self) -> int:
        return self.heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.kv_heads * self.head_dim


LLAMA3_8B = LlamaConfig()


class DeviceBuffer:
    """Device memory from the library's allocator (skainet_hip_malloc), with numpy upload / download."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        self.ptr = _lib.hip().skainet_hip_malloc(self.nbytes)
        if not self.ptr:
            raise HipError("malloc: " + _lib.last_error())

    def data_ptr(self) -> int:
        return self.ptr

    def at(self, byte_offset: int) -> int:
        return self.ptr + int(byte_offset)

    def upload(self, a: np.ndarray, byte_offset: int = 0) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        check(_lib.hip().skainet_hip_memcpy_h2d(self.ptr + byte_offset, a.ctypes.data, a.nbytes), "h2d")
        return self

    def download(self, dtype, count: int, byte_offset: int = 0) -> np.ndarray:
        out = np.empty(count, dtype=dtype)
        check(_lib.hip().skainet_hip_memcpy_d2h(out.ctypes.data, self.ptr + byte_offset, out.nbytes), "d2h")
        return out

    def close(self) -> None:
        if self.ptr:
            _lib.hip().skainet_hip_free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


@dataclass
class LayerWeights:
    attn_norm: DeviceBuffer      # fp32 [hidden]
    wqkv: kernels.DeviceWeight   # [(heads + 2 kv_heads) * head_dim, hidden]
    wo: kernels.DeviceWeight     # [hidden, heads * head_dim]
    ffn_norm: DeviceBuffer       # fp32 [hidden]
    w_gate_up: kernels.DeviceWeight   # [2 * ffn, hidden], row 2j = gate row j, row 2j + 1 = up row j
    w_down: kernels.DeviceWeight      # [hidden, ffn]


class LlamaWeights:
    """Random-init weights of the architecture, quantised on the host and resident on the device.

    `host` keeps the packed bytes and norm gains when `keep_host` is set, so a CPU checker can consume the very
    same bytes."""

    def __init__(self, cfg: LlamaConfig, seed: int = 0, sigma: float = 0.02, keep_host: bool = False, progress=None,
                 distinct_layers: int = 0):
        """distinct_layers > 0: only that many layers get values of their own; layer i re-uses the packed bytes of
        layer i % distinct_layers in a device allocation of its own (same HBM traffic, far less host-side
        generation and quantisation time for a benchmark)."""
        kernels._require_available()
        self.cfg = cfg
        self.host = {} if keep_host else None
        rng = np.random.default_rng(seed)
        bytes_of = {}

        def packed(name, enc, rows, cols, same_as=None):
            if same_as is not None:
                return kernels.DeviceWeight.upload(enc, bytes_of[same_as], rows, cols)
            # generated and quantised in row chunks so the fp32 source never exceeds ~256 MB
            _, bs, nb = kernels.ENCODINGS[enc]
            out = np.empty(rows * (cols // bs) * nb, dtype=np.uint8)
            step = max(1, (64 << 20) // cols)
            row_bytes = (cols // bs) * nb
            for r0 in range(0, rows, step):
                r1 = min(rows, r0 + step)
                w = rng.standard_normal((r1 - r0, cols), dtype=np.float32) * np.float32(sigma)
                out[r0 * row_bytes:r1 * row_bytes] = kernels.quantize(enc, w)
            if self.host is not None:
                self.host[name] = out
            if distinct_layers > 0:
                bytes_of[name] = out
            if progress:
                progress(name)
            return kernels.DeviceWeight.upload(enc, out, rows, cols)

        def gain(name, same_as=None):
            if same_as is not None:
                return DeviceBuffer(bytes_of[same_as].nbytes).upload(bytes_of[same_as])
            g = (1.0 + 0.1 * rng.standard_normal(cfg.hidden)).astype(np.float32)
            if distinct_layers > 0:
                bytes_of[name] = g
            if self.host is not None:
                self.host[name] = g
            return DeviceBuffer(g.nbytes).upload(g)

        le = cfg.linear_encoding
        self.tok_embd = packed("tok_embd", le, cfg.vocab, cfg.hidden)
        self.layers: List[LayerWeights] = []
        for i in range(cfg.layers):
            src = None if distinct_layers <= 0 or i < distinct_layers else f"l{i % distinct_layers}"

            def same(part):
                return None if src is None else f"{src}.{part}"

            self.layers.append(LayerWeights(
                attn_norm=gain(f"l{i}.attn_norm", same("attn_norm")),
                wqkv=packed(f"l{i}.wqkv", le, cfg.q_dim + 2 * cfg.kv_dim, cfg.hidden, same("wqkv")),
                wo=packed(f"l{i}.wo", le, cfg.hidden, cfg.q_dim, same("wo")),
                ffn_norm=gain(f"l{i}.ffn_norm", same("ffn_norm")),
                w_gate_up=packed(f"l{i}.w_gate_up", le, 2 * cfg.ffn, cfg.hidden, same("w_gate_up")),
                w_down=packed(f"l{i}.w_down", le, cfg.hidden, cfg.ffn, same("w_down")),
            ))
        self.out_norm = gain("out_norm")
        self.head = packed("head", cfg.head_encoding, cfg.vocab, cfg.hidden)

    # ------------------------------------------------------------------ GGUF files
    @classmethod
    def from_gguf(cls, path: str, ctx_max: Optional[int] = None, keep_host: bool = False) -> "LlamaWeights":
        """Load a llama-architecture GGUF file (llama.cpp tensor names): packed tensors go from the file mapping to the
        device; q/k/v are concatenated and gate/up interleaved row by row on the way (they must share an encoding).
        `output.weight` may be absent (tied embeddings): the token embedding is used."""
        from . import gguf
        kernels._require_available()
        with gguf.GGUFReader(path) as r:
            f = r.fields
            arch = f.get("general.architecture", "llama")

            def meta(key, default=None):
                v = f.get(f"{arch}.{key}", default)
                if v is None:
                    raise gguf.GGUFError(f"{path}: metadata key {arch}.{key} is missing")
                return v

            hidden, heads = int(meta("embedding_length")), int(meta("attention.head_count"))
            emb = r.info("token_embd.weight")
            cfg = LlamaConfig(
                layers=int(meta("block_count")), hidden=hidden, heads=heads,
                kv_heads=int(meta("attention.head_count_kv", heads)),
                head_dim=int(meta("attention.key_length", hidden // heads)), ffn=int(meta("feed_forward_length")),
                vocab=emb.rows, rms_eps=float(meta("attention.layer_norm_rms_epsilon", 1e-5)),
                rope_theta=float(meta("rope.freq_base", 10000.0)),
                ctx_max=int(ctx_max if ctx_max is not None else meta("context_length", 2048)),
                linear_encoding=r.info("blk.0.attn_q.weight").type_name,
                head_encoding=(r.info("output.weight") if "output.weight" in r.names() else emb).type_name)
            self = object.__new__(cls)
            self.cfg = cfg
            self.host = {} if keep_host else None

            def keep(name, a):
                if self.host is not None:
                    self.host[name] = np.array(a)
                return a

            def packed_rows(name, rows_expected, cols_expected):
                t = r.info(name)
                if t.type_name not in gguf.DEVICE_ENCODINGS:
                    raise gguf.GGUFError(f"{path}: {name} is {t.type_name}; the device kernels take {gguf.DEVICE_ENCODINGS}")
                if (t.rows, t.cols) != (rows_expected, cols_expected):
                    raise gguf.GGUFError(f"{path}: {name} is {t.rows} x {t.cols}, expected {rows_expected} x {cols_expected}")
                return t.type_name, r.tensor_bytes(name).reshape(t.rows, -1)

            def fused(name, parts, interleave=False):
                encs = {e for e, _ in parts}
                if len(encs) != 1:
                    raise gguf.GGUFError(f"{path}: {name}: tensors fused into one product must share an encoding, got {sorted(encs)}")
                mats = [m for _, m in parts]
                if interleave:
                    out = np.empty((2 * mats[0].shape[0], mats[0].shape[1]), np.uint8)
                    out[0::2], out[1::2] = mats
                else:
                    out = np.concatenate(mats, axis=0)
                out = keep(name, out.reshape(-1))
                return kernels.DeviceWeight.upload(encs.pop(), out, sum(m.shape[0] for m in mats), cfg_cols[name.split(".")[-1]])

            def single(name, host_name, rows, cols):
                enc, m = packed_rows(name, rows, cols)
                return kernels.DeviceWeight.upload(enc, keep(host_name, m.reshape(-1)), rows, cols)

            def gain(name, host_name):
                g = np.ascontiguousarray(r.tensor_f32(name), dtype=np.float32).reshape(-1)
                if g.size != hidden:
                    raise gguf.GGUFError(f"{path}: {name} has {g.size} elements, expected {hidden}")
                return DeviceBuffer(g.nbytes).upload(keep(host_name, g))

            cfg_cols = {"wqkv": hidden, "w_gate_up": hidden}
            self.tok_embd = single("token_embd.weight", "tok_embd", cfg.vocab, hidden)
            self.layers = []
            for i in range(cfg.layers):
                b = f"blk.{i}."
                self.layers.append(LayerWeights(
                    attn_norm=gain(b + "attn_norm.weight", f"l{i}.attn_norm"),
                    wqkv=fused(f"l{i}.wqkv", [packed_rows(b + "attn_q.weight", cfg.q_dim, hidden),
                                              packed_rows(b + "attn_k.weight", cfg.kv_dim, hidden),
                                              packed_rows(b + "attn_v.weight", cfg.kv_dim, hidden)]),
                    wo=single(b + "attn_output.weight", f"l{i}.wo", hidden, cfg.q_dim),
                    ffn_norm=gain(b + "ffn_norm.weight", f"l{i}.ffn_norm"),
                    w_gate_up=fused(f"l{i}.w_gate_up", [packed_rows(b + "ffn_gate.weight", cfg.ffn, hidden),
                                                        packed_rows(b + "ffn_up.weight", cfg.ffn, hidden)], interleave=True),
                    w_down=single(b + "ffn_down.weight", f"l{i}.w_down", hidden, cfg.ffn)))
            self.out_norm = gain("output_norm.weight", "out_norm")
            head_name = "output.weight" if "output.weight" in r.names() else "token_embd.weight"
            self.head = single(head_name, "head", cfg.vocab, hidden)
        return self

    def to_gguf(self, path: str) -> None:
        """Write this model as a llama-architecture GGUF file with llama.cpp tensor names (needs keep_host=True)."""
        from . import gguf
        if self.host is None:
            raise ValueError("to_gguf needs the host copies: build the weights with keep_host=True")
        c, h = self.cfg, self.host
        w = gguf.GGUFWriter()
        w.add_string("general.architecture", "llama")
        for key, v in (("block_count", c.layers), ("embedding_length", c.hidden), ("attention.head_count", c.heads),
                       ("attention.head_count_kv", c.kv_heads), ("attention.key_length", c.head_dim),
                       ("feed_forward_length", c.ffn), ("context_length", c.ctx_max), ("vocab_size", c.vocab)):
            w.add_u32("llama." + key, v)
        w.add_f32("llama.attention.layer_norm_rms_epsilon", c.rms_eps)
        w.add_f32("llama.rope.freq_base", c.rope_theta)
        le, he = c.linear_encoding, c.head_encoding
        _, bs, nb = kernels.ENCODINGS[le]
        row_bytes = c.hidden // bs * nb
        w.add_tensor("token_embd.weight", le, (c.vocab, c.hidden), h["tok_embd"])
        for i in range(c.layers):
            b = f"blk.{i}."
            qkv = h[f"l{i}.wqkv"].reshape(-1, row_bytes)
            gu = h[f"l{i}.w_gate_up"].reshape(-1, row_bytes)
            w.add_tensor(b + "attn_norm.weight", "F32", (c.hidden,), h[f"l{i}.attn_norm"])
            w.add_tensor(b + "attn_q.weight", le, (c.q_dim, c.hidden), qkv[:c.q_dim])
            w.add_tensor(b + "attn_k.weight", le, (c.kv_dim, c.hidden), qkv[c.q_dim:c.q_dim + c.kv_dim])
            w.add_tensor(b + "attn_v.weight", le, (c.kv_dim, c.hidden), qkv[c.q_dim + c.kv_dim:])
            w.add_tensor(b + "attn_output.weight", le, (c.hidden, c.q_dim), h[f"l{i}.wo"])
            w.add_tensor(b + "ffn_norm.weight", "F32", (c.hidden,), h[f"l{i}.ffn_norm"])
            w.add_tensor(b + "ffn_gate.weight", le, (c.ffn, c.hidden), gu[0::2])
            w.add_tensor(b + "ffn_up.weight", le, (c.ffn, c.hidden), gu[1::2])
            w.add_tensor(b + "ffn_down.weight", le, (c.hidden, c.ffn), h[f"l{i}.w_down"])
        w.add_tensor("output_norm.weight", "F32", (c.hidden,), h["out_norm"])
        w.add_tensor("output.weight", he, (c.vocab, c.hidden), h["head"])
        w.write(path)

    def packed_bytes(self) -> int:
        n = self.tok_embd.nbytes + self.head.nbytes
        for l in self.layers:
            n += l.wqkv.nbytes + l.wo.nbytes + l.w_gate_up.nbytes + l.w_down.nbytes
        return n

    def decode_bytes_per_token(self, context: int) -> int:
        """Algorithmic HBM bytes of one decode step: every linear weight and the head once, the KV cache up to `context`."""
        c = self.cfg
        return (self.packed_bytes() - self.tok_embd.nbytes) + 2 * c.layers * c.kv_heads * context * c.head_dim * 4


class LlamaDecoder:
    """Prefill + greedy decode for batch 1, state (KV cache, position, current token) on the device."""

    def __init__(self, weights: LlamaWeights, max_prefill: int = 512):
        c = self.cfg = weights.cfg
        self.w = weights
        self.max_rows = max(1, max_prefill)
        f = 4
        rows = self.max_rows
        self.h = DeviceBuffer(rows * c.hidden * f)
        self.norm = DeviceBuffer(rows * c.hidden * f)
        self.qkv = DeviceBuffer(rows * (c.q_dim + 2 * c.kv_dim) * f)
        self.q = DeviceBuffer(rows * c.q_dim * f)            # [heads, rows, head_dim]
        self.attn = DeviceBuffer(rows * c.q_dim * f)         # [heads, rows, head_dim]
        self.attn_rows = DeviceBuffer(rows * c.q_dim * f)    # [rows, heads * head_dim]
        self.act = DeviceBuffer(rows * c.ffn * f)
        self.logits = DeviceBuffer(c.vocab * f)
        self.kv_layer_floats = c.kv_heads * c.ctx_max * c.head_dim
        self.k_cache = DeviceBuffer(c.layers * self.kv_layer_floats * f)
        self.v_cache = DeviceBuffer(c.layers * self.kv_layer_floats * f)
        self.pos = DeviceBuffer(4).upload(np.zeros(1, np.int32))        # tokens already in the cache
        self.kv_len = DeviceBuffer(4).upload(np.zeros(1, np.int32))     # = pos + 1 during a decode step
        self.token = DeviceBuffer(4).upload(np.zeros(1, np.int32))
        self.rope_table = DeviceBuffer(4 * c.head_dim)      # (cos, sin) per rotation pair of the current decode position
        self.generated = DeviceBuffer(4 * (c.ctx_max + 1))   # generated[p] = the token predicted for position p
        self.prompt_len = 0
        self._graph: Optional[kernels.Graph] = None
        self._graph_bound = 0          # key count the recorded step was laid out for (its attention splits that many keys)
        self._host_pos = 0             # the device-side position, tracked on the host so a replay needs no read-back

    # ------------------------------------------------------------------ building blocks
    def _block(self, li: int, rows: int, pos_start: int, pos_dev, seq_kv: int, kv_len_dev) -> None:
        """One decoder block over `rows` token rows already in self.h. Prefill: positions pos_start.., K/V rows
        written at those positions, causal attention over seq_kv = pos_start + rows keys. Decode: one row at the
        device-side position, attention over the whole cache bounded by the device-side key length."""
        c, w, L = self.cfg, self.w, self.w.layers[li]
        f = 4
        kx = kernels
        kc = self.k_cache.at(li * self.kv_layer_floats * f)
        vc = self.v_cache.at(li * self.kv_layer_floats * f)
        if rows == 1 and pos_dev is not None:
            # decode: norm, projection, RoPE and the cache append are one launch
            L.wqkv.matmul_qkv_rope(self.h, self.q, kc, vc, c.heads, c.kv_heads, c.head_dim, c.ctx_max, pos_dev,
                                   c.rope_theta, gain=L.attn_norm, eps=c.rms_eps, rope_table=self.rope_table)
        else:
            L.wqkv.matmul_fused(self.h, rows, self.qkv, gain=L.attn_norm, eps=c.rms_eps)
            # rotated queries to [heads, rows, head_dim]; rotated keys and raw values into the cache rows of these positions
            kx.rope_qkv_dev(self.qkv, self.q, kc, vc, rows, c.heads, c.kv_heads, c.head_dim, c.ctx_max, pos_start, pos_dev,
                            c.rope_theta)
        scale = float(1.0 / np.sqrt(c.head_dim))
        if rows == 1 and pos_dev is not None:
            # one token: [heads, 1, head_dim] is already the projection's input row; attention and projection as a pair
            L.wo.attn_out_proj(self.q, kc, vc, c.heads, c.kv_heads, c.head_dim, seq_kv, c.ctx_max, scale, self.h, self.attn,
                               residual=self.h, lengths=kv_len_dev)
        else:
            # attention straight into token rows: what the output projection multiplies
            kx.sdpa_cache_rows_dev(self.q, kc, vc, self.attn_rows, 1, c.heads, c.kv_heads, rows, seq_kv, c.ctx_max, c.head_dim, scale,
                                   True, 0, 0, kv_len_dev)
            L.wo.matmul_fused(self.attn_rows, rows, self.h, residual=self.h, epilogue=kx.EPI_RESIDUAL)
        if rows > 8:
            # prompt rows: the block in one call (the SwiGLU rides in the down projection's rounding pass)
            L.w_gate_up.mlp_swiglu(L.w_down, self.h, rows, self.h, gain=L.ffn_norm, eps=c.rms_eps, residual=self.h)
        else:
            L.w_gate_up.matmul_fused(self.h, rows, self.act, gain=L.ffn_norm, eps=c.rms_eps, epilogue=kx.EPI_SWIGLU)
            L.w_down.matmul_fused(self.act, rows, self.h, residual=self.h, epilogue=kx.EPI_RESIDUAL)

    def _head(self, row: int) -> None:
        c = self.cfg
        kernels.rms_norm_dev(self.h.at(4 * row * c.hidden), self.w.out_norm, self.norm, 1, c.hidden, c.rms_eps)
        self.w.head.matmul(self.norm, 1, self.logits)
        kernels.argmax_rows_dev(self.logits, 1, c.vocab, self.token)

    # ------------------------------------------------------------------ public API
    def prefill(self, token_ids) -> int:
        """Run the prompt through the stack, fill the KV cache, return the greedy next token."""
        c = self.cfg
        ids64 = np.ascontiguousarray(token_ids, dtype=np.int64).reshape(-1)
        rows = int(ids64.size)
        if rows < 1 or rows > self.max_rows or rows > c.ctx_max:
            raise ValueError(f"prompt of {rows} tokens does not fit (max_prefill {self.max_rows}, ctx {c.ctx_max})")
        if ids64.min() < 0 or ids64.max() >= c.vocab:       # the gather reads embedding rows by id: checked before any launch
            bad = ids64[(ids64 < 0) | (ids64 >= c.vocab)][0]
            raise ValueError(f"token id {int(bad)} is outside the vocabulary [0, {c.vocab})")
        ids = ids64.astype(np.int32)
        ids_dev = DeviceBuffer(ids.nbytes).upload(ids)
        self.w.tok_embd.dequantize_rows(ids_dev, rows, self.h)
        for li in range(c.layers):
            self._block(li, rows, 0, None, rows, None)
        self._head(rows - 1)
        kernels.sync()
        self.pos.upload(np.array([rows], np.int32))
        self.kv_len.upload(np.array([rows + 1], np.int32))
        self.prompt_len = rows
        self._host_pos = rows
        kernels.i32_store_at_dev(self.generated, self.pos, 0, self.token)
        kernels.sync()
        ids_dev.close()
        return int(self.token.download(np.int32, 1)[0])

    KEY_BUCKET = 512

    def _key_bound(self, keys: int) -> int:
        """The key count a step is laid out for: the next multiple of KEY_BUCKET (the device-side length picks the keys
        that exist, the bound decides how attention splits them)."""
        b = self.KEY_BUCKET
        return min(self.cfg.ctx_max, (keys + b - 1) // b * b)

    def _decode_step(self, bound: Optional[int] = None) -> None:
        """Consumes self.token at device position self.pos, leaves the next token in self.token, advances the position."""
        c = self.cfg
        if bound is None:
            bound = self._key_bound(self._host_pos + 1)
        self.w.tok_embd.dequantize_rows(self.token, 1, self.h)
        kernels.rope_table_dev(self.pos, c.rope_theta, c.head_dim, self.rope_table)     # once per token, shared by all layers
        for li in range(c.layers):
            self._block(li, 1, 0, self.pos, bound, self.kv_len)
        self._head(0)
        kernels.decode_advance_dev(self.pos, self.kv_len, self.token, self.generated, c.ctx_max)

    def _graph_step(self) -> None:
        """One decode step through the recorded graph; records it first (one eager step, then the recording, which runs
        nothing) when there is none, when the library's scratch moved since, or when the cache outgrew its key bound."""
        keys = self._host_pos + 1
        if self._graph is not None and (not self._graph.valid() or keys > self._graph_bound):
            self._graph.close()
            self._graph = None
        if self._graph is None:
            bound = self._key_bound(keys + 1)          # the recording serves the steps after this one
            self._decode_step(bound)                   # eager once: sizes every scratch buffer
            kernels.sync()
            self._host_pos += 1
            if self._host_pos < self.cfg.ctx_max:      # at the limit there is no next step to record
                with kernels.Graph() as g:
                    self._decode_step(bound)
                self._graph, self._graph_bound = g, bound
            return
        self._graph.launch()
        self._host_pos += 1

    def run_steps(self, steps: int, use_graph: bool = True) -> None:
        """`steps` decode steps back to back without reading anything back (tokens feed back on the device)."""
        if self._host_pos + steps > self.cfg.ctx_max:
            raise ValueError(f"{steps} more tokens would pass the context limit {self.cfg.ctx_max}")
        for _ in range(steps):
            if use_graph:
                self._graph_step()
            else:
                self._decode_step()
                self._host_pos += 1

    def decode(self, steps: int, use_graph: bool = True) -> np.ndarray:
        """Greedy-decode `steps` tokens after prefill(); returns them. With use_graph the step is recorded once per key
        bucket and replayed."""
        c = self.cfg
        if self._host_pos + steps > c.ctx_max:
            raise ValueError(f"{steps} more tokens would pass the context limit {c.ctx_max}")
        out = np.empty(steps, np.int32)
        for i in range(steps):
            self.run_steps(1, use_graph)
            kernels.sync()
            out[i] = int(self.token.download(np.int32, 1)[0])
        return out

    def decode_timed(self, steps: int) -> float:
        """`steps` recorded steps without reading tokens back; returns seconds (host clock around launch + sync). Tokens
        stay on the device (greedy feedback happens there)."""
        import time
        if self._host_pos + steps > self.cfg.ctx_max:
            raise ValueError(f"{steps} more tokens would pass the context limit {self.cfg.ctx_max}")
        kernels.sync()
        t0 = time.perf_counter()
        self.run_steps(steps)
        kernels.sync()
        return time.perf_counter() - t0

    def close(self) -> None:
        """Free the recorded decode graph (device buffers go with their owners)."""
        if self._graph is not None:
            self._graph.close()
            self._graph = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def generated_tokens(self) -> np.ndarray:
        """Every token emitted since the last prefill (the prefill's own next-token first), read from the device log."""
        n = self.position() - self.prompt_len + 1
        return self.generated.download(np.int32, n, 4 * self.prompt_len)

    def position(self) -> int:
        return int(self.pos.download(np.int32, 1)[0])

    def last_logits(self) -> np.ndarray:
        return self.logits.download(np.float32, self.cfg.vocab)

    def hidden_rows(self, rows: int) -> np.ndarray:
        return self.h.download(np.float32, rows * self.cfg.hidden).reshape(rows, self.cfg.hidden)
