"""The decoder's CPU checker checked against itself (no GPU): feeding a prompt at once and token by token must give
the same state (KV-cache consistency and the causal rule), RoPE must be a pure rotation that composes additively
in the position, and a rotation-free single-layer case must reduce to plain matrix algebra."""
import numpy as np

from decoder_check import CheckDecoder
from skainet_amd import kernels
from skainet_amd.decoder import LlamaConfig


def tiny(layers=2):
    cfg = LlamaConfig(layers=layers, hidden=256, heads=4, kv_heads=2, head_dim=64, ffn=512, vocab=300, ctx_max=32,
                      rope_theta=10000.0)
    rng = np.random.default_rng(0)
    host = {}

    def pk(name, enc, r, c):
        host[name] = kernels.quantize(enc, (rng.standard_normal((r, c)) * 0.05).astype(np.float32))

    pk("tok_embd", "Q4_K", cfg.vocab, cfg.hidden)
    pk("head", "Q6_K", cfg.vocab, cfg.hidden)
    host["out_norm"] = (1 + 0.1 * rng.standard_normal(cfg.hidden)).astype(np.float32)
    for i in range(layers):
        host[f"l{i}.attn_norm"] = (1 + 0.1 * rng.standard_normal(cfg.hidden)).astype(np.float32)
        host[f"l{i}.ffn_norm"] = (1 + 0.1 * rng.standard_normal(cfg.hidden)).astype(np.float32)
        pk(f"l{i}.wqkv", "Q4_K", cfg.q_dim + 2 * cfg.kv_dim, cfg.hidden)
        pk(f"l{i}.wo", "Q4_K", cfg.hidden, cfg.q_dim)
        pk(f"l{i}.w_gate_up", "Q4_K", 2 * cfg.ffn, cfg.hidden)
        pk(f"l{i}.w_down", "Q4_K", cfg.hidden, cfg.ffn)
    return cfg, host


def test_incremental_equals_full():
    cfg, host = tiny()
    ids = [3, 5, 7, 11, 13, 299]
    a, b = CheckDecoder(cfg, host), CheckDecoder(cfg, host)
    h, logits = a.forward(ids)
    for t in ids:
        h1, logits1 = b.forward([t])
    assert np.abs(logits - logits1).max() < 1e-10
    assert np.abs(h[-1] - h1[-1]).max() < 1e-10
    assert a.k[1].shape == (cfg.kv_heads, len(ids), cfg.head_dim)
    assert np.abs(a.k[1] - b.k[1]).max() < 1e-12


def test_rope_is_a_rotation_and_composes():
    cfg, host = tiny(1)
    c = CheckDecoder(cfg, host)
    x = np.random.default_rng(1).standard_normal((3, cfg.heads, cfg.head_dim))
    y = c.rope(x, 5)
    pair_norm = lambda z: z[..., 0::2] ** 2 + z[..., 1::2] ** 2
    assert np.allclose(pair_norm(x), pair_norm(y))
    assert np.allclose(c.rope(x, 0)[0], x[0])                    # position 0 is the identity
    assert np.allclose(c.rope(c.rope(x[:1], 3), 4), c.rope(x[:1], 7))
    # dot products depend on the position difference only
    q, k = x[:1, :1], x[1:2, :1]
    d1 = (c.rope(q, 9) * c.rope(k, 4)).sum()
    d2 = (c.rope(q, 25) * c.rope(k, 20)).sum()
    assert np.isclose(d1, d2)


def test_single_token_reduces_to_matrix_algebra():
    """One token at position 0: RoPE is the identity and attention over one key returns its value row."""
    cfg, host = tiny(1)
    c = CheckDecoder(cfg, host)
    h, _ = c.forward([42])
    L = c.layers[0]
    x0 = c.tok[42]
    n1 = x0 / np.sqrt((x0 ** 2).mean() + cfg.rms_eps) * L["attn_norm"]
    v = (L["wqkv"] @ n1)[cfg.q_dim + cfg.kv_dim:].reshape(cfg.kv_heads, cfg.head_dim)
    att = np.repeat(v, cfg.heads // cfg.kv_heads, axis=0).reshape(-1)
    h1 = x0 + L["wo"] @ att
    n2 = h1 / np.sqrt((h1 ** 2).mean() + cfg.rms_eps) * L["ffn_norm"]
    gu = L["w_gate_up"] @ n2
    g, u = gu[0::2], gu[1::2]
    want = h1 + L["w_down"] @ (g / (1 + np.exp(-g)) * u)
    assert np.abs(h[0] - want).max() < 1e-10
