"""CPU checker for the Llama-shaped decoder: the same block arithmetic in float64 numpy over the very same packed
weight bytes (decoded by the oracle's bit-exact dequantisers). Test infrastructure only."""
import numpy as np

from oracle import lib as O


class CheckDecoder:
    def __init__(self, cfg, host):
        """`host`: name -> packed bytes / fp32 gain, as LlamaWeights(keep_host=True).host holds them."""
        self.cfg = c = cfg
        le, he = c.linear_encoding, c.head_encoding

        def mat(name, enc, rows, cols):
            return O.dequant(enc, host[name]).reshape(rows, cols).astype(np.float64)

        self.tok = mat("tok_embd", le, c.vocab, c.hidden)
        self.head = mat("head", he, c.vocab, c.hidden)
        self.out_norm = host["out_norm"].astype(np.float64)
        self.layers = []
        for i in range(c.layers):
            self.layers.append(dict(
                attn_norm=host[f"l{i}.attn_norm"].astype(np.float64),
                wqkv=mat(f"l{i}.wqkv", le, c.q_dim + 2 * c.kv_dim, c.hidden),
                wo=mat(f"l{i}.wo", le, c.hidden, c.q_dim),
                ffn_norm=host[f"l{i}.ffn_norm"].astype(np.float64),
                w_gate_up=mat(f"l{i}.w_gate_up", le, 2 * c.ffn, c.hidden),
                w_down=mat(f"l{i}.w_down", le, c.hidden, c.ffn)))
        self.k = [np.zeros((c.kv_heads, 0, c.head_dim)) for _ in range(c.layers)]
        self.v = [np.zeros((c.kv_heads, 0, c.head_dim)) for _ in range(c.layers)]

    def _rms(self, x, g):
        return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + self.cfg.rms_eps) * g

    def rope(self, x, pos0):
        """x [tokens, heads, head_dim]: adjacent pairs rotated by (pos0 + t) * theta^(-2i / head_dim)."""
        c = self.cfg
        t = np.arange(x.shape[0], dtype=np.float64)[:, None, None] + pos0
        i = np.arange(c.head_dim // 2, dtype=np.float64)[None, None, :]
        ang = t * c.rope_theta ** (-2.0 * i / c.head_dim)
        a, b = x[..., 0::2], x[..., 1::2]
        out = np.empty_like(x)
        out[..., 0::2] = a * np.cos(ang) - b * np.sin(ang)
        out[..., 1::2] = a * np.sin(ang) + b * np.cos(ang)
        return out

    def forward(self, token_ids):
        """Feeds the tokens at the positions after everything already cached; returns (hidden rows, logits of the last)."""
        c = self.cfg
        ids = np.asarray(token_ids, dtype=np.int64)
        n = ids.size
        pos0 = self.k[0].shape[1]
        h = self.tok[ids].copy()
        per = c.heads // c.kv_heads
        for li, L in enumerate(self.layers):
            x = self._rms(h, L["attn_norm"])
            qkv = x @ L["wqkv"].T
            q = self.rope(qkv[:, :c.q_dim].reshape(n, c.heads, c.head_dim), pos0)
            k = self.rope(qkv[:, c.q_dim:c.q_dim + c.kv_dim].reshape(n, c.kv_heads, c.head_dim), pos0)
            v = qkv[:, c.q_dim + c.kv_dim:].reshape(n, c.kv_heads, c.head_dim)
            self.k[li] = np.concatenate([self.k[li], k.transpose(1, 0, 2)], axis=1)
            self.v[li] = np.concatenate([self.v[li], v.transpose(1, 0, 2)], axis=1)
            att = np.empty((n, c.heads, c.head_dim))
            for hh in range(c.heads):
                kk, vv = self.k[li][hh // per], self.v[li][hh // per]
                s = (q[:, hh, :] @ kk.T) / np.sqrt(c.head_dim)
                key = np.arange(kk.shape[0])[None, :]
                s = np.where(key <= (pos0 + np.arange(n))[:, None], s, -np.inf)
                s -= s.max(axis=1, keepdims=True)
                p = np.exp(s)
                att[:, hh, :] = (p / p.sum(axis=1, keepdims=True)) @ vv
            h = h + att.reshape(n, c.q_dim) @ L["wo"].T
            x = self._rms(h, L["ffn_norm"])
            gu = x @ L["w_gate_up"].T
            g, u = gu[:, 0::2], gu[:, 1::2]          # rows of w_gate_up alternate gate row, up row
            h = h + (g / (1.0 + np.exp(-g)) * u) @ L["w_down"].T
        logits = self._rms(h[-1], self.out_norm) @ self.head.T
        return h, logits
