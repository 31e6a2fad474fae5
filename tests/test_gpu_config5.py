"""The synthetic Llama-3-8B-shape decoder stack at its real shapes: 32 layers, hidden 4096, 32 / 8 heads of 128, SwiGLU
FFN 14336, vocabulary 128256, Q4_K linears and a Q6_K head, prefill of 512 tokens and greedy decode into a context
above 1024.

The stack has no counterpart in the reference (parity unpinned by construction): every check is against float64
arithmetic on the very same packed bytes, decoded by the oracle's bit-exact dequantisers. At this size the whole stack
cannot be replayed in float64 (7 G weights), so the full-size model is checked launch by launch on its own live state
-- the 128256 x 4096 Q6_K head, the fused 28672 x 4096 RMSNorm + gate/up + SwiGLU launch, the 6144 x 4096 q/k/v
projection with RMSNorm, RoPE and cache append, attention over more than 1024 cached keys -- and a 2-layer model at
the full widths is teacher-forced against the float64 checker end to end.
Tolerances: fp32 routes 1e-3 of the largest reference magnitude, the bf16-operand MFMA prefill 2e-2."""
import numpy as np
import pytest

from decoder_check import CheckDecoder
from oracle import lib as O

pytestmark = pytest.mark.gpu

PROMPT = 512
DECODED = 530                       # context 1042 at the end


def max_norm_err(got, ref):
    ref = np.asarray(ref, np.float64)
    return float(np.abs(np.asarray(got, np.float64) - ref).max() / max(np.abs(ref).max(), 1e-30))


def rms(x, g, eps):
    x = np.asarray(x, np.float64)
    return x / np.sqrt((x * x).mean() + eps) * np.asarray(g, np.float64)


def packed_rows(host, name, enc, cols, rows):
    """fp64 [len(rows), cols] of the given rows of a packed host weight."""
    from skainet_amd.kernels import ENCODINGS
    _, bs, nb = ENCODINGS[enc]
    rb = cols // bs * nb
    m = host[name].reshape(-1, rb)
    return O.dequant(enc, np.ascontiguousarray(m[rows]).reshape(-1)).reshape(len(rows), cols).astype(np.float64)


@pytest.fixture(scope="module")
def full_stack(hip_backend):
    """32 layers at the real shapes, 4 layers of distinct values (layer i carries the bytes of layer i % 4 in an
    allocation of its own), prefilled with 512 tokens and decoded by replaying the recorded 32-layer step."""
    from skainet_amd.decoder import LLAMA3_8B, LlamaDecoder, LlamaWeights
    cfg = LLAMA3_8B
    w = LlamaWeights(cfg, seed=2048, keep_host=True, distinct_layers=4)
    dec = LlamaDecoder(w, max_prefill=PROMPT)
    prompt = np.random.default_rng(5).integers(0, cfg.vocab, PROMPT)
    first = dec.prefill(prompt)
    toks = dec.decode(DECODED, use_graph=True)
    yield cfg, w, dec, prompt, first, toks
    dec.close()


def test_stack_reaches_a_long_context_and_stays_sane(full_stack):
    cfg, w, dec, prompt, first, toks = full_stack
    assert dec.position() == PROMPT + DECODED > 1024
    gen = dec.generated_tokens()
    assert gen[0] == first and np.array_equal(gen[1:], toks)
    assert ((toks >= 0) & (toks < cfg.vocab)).all()
    logits = dec.last_logits()
    assert np.isfinite(logits).all() and int(np.argmax(logits)) == int(toks[-1])
    h = dec.hidden_rows(1)
    assert np.isfinite(h).all() and np.abs(h).max() < 1e4


def test_replayed_32_layer_step_equals_the_eager_step(full_stack):
    """The recorded graph and the eager launches are the same kernels on the same state: identical tokens."""
    from skainet_amd.decoder import LlamaDecoder
    cfg, w, dec, prompt, first, toks = full_stack
    ref = LlamaDecoder(w, max_prefill=PROMPT)
    assert ref.prefill(prompt) == first
    assert np.array_equal(ref.decode(6, use_graph=False), toks[:6])
    ref.close()


def test_q6k_head_128256_rows_on_the_live_hidden_state(full_stack):
    cfg, w, dec, *_ = full_stack
    h = dec.hidden_rows(1)[0]
    xn = rms(h, w.host["out_norm"], cfg.rms_eps)
    logits = dec.last_logits()
    blocks = [0, 31744, 64000, 99968, 128000, cfg.vocab - 64]          # six blocks of 64 vocabulary rows
    rows = np.concatenate([np.arange(b, b + 64) for b in blocks])
    want = packed_rows(w.host, "head", cfg.head_encoding, cfg.hidden, rows) @ xn
    scale = np.abs(logits).max()
    assert np.abs(logits[rows] - want).max() <= 1e-3 * scale


@pytest.mark.parametrize("layer", [3, 17])
def test_fused_gate_up_28672_rows_with_norm_and_swiglu(full_stack, torch_cuda, layer):
    cfg, w, dec, *_ = full_stack
    torch = torch_cuda
    L = w.layers[layer]
    h = dec.hidden_rows(1)[0]
    act = torch.full((cfg.ffn,), 7.0, device="cuda")
    L.w_gate_up.matmul_fused(dec.h, 1, act, gain=L.ffn_norm, eps=cfg.rms_eps, epilogue=1 + 1)      # EPI_SWIGLU
    from skainet_amd import kernels
    kernels.sync()
    src = f"l{layer % 4}"
    xn = rms(h, w.host[f"{src}.ffn_norm"], cfg.rms_eps)
    chans = np.concatenate([np.arange(c0, c0 + 32) for c0 in (0, 2048, 5000, 7168, 9999, 12000, 14000, cfg.ffn - 32)])
    rows = np.stack([2 * chans, 2 * chans + 1], 1).reshape(-1)
    p = packed_rows(w.host, f"{src}.w_gate_up", cfg.linear_encoding, cfg.hidden, rows) @ xn
    g, u = p[0::2], p[1::2]
    want = g / (1 + np.exp(-g)) * u
    got = act.cpu().numpy()
    assert np.isfinite(got).all()
    assert np.abs(got[chans] - want).max() <= 1e-3 * max(np.abs(want).max(), np.abs(got).max())


@pytest.mark.parametrize("layer", [2, 31])
def test_qkv_6144_rows_with_norm_rope_and_cache_append(full_stack, torch_cuda, layer):
    from skainet_amd import kernels
    cfg, w, dec, *_ = full_stack
    torch = torch_cuda
    L = w.layers[layer]
    pos = dec.position()
    h = dec.hidden_rows(1)[0]
    q = torch.zeros(cfg.q_dim, device="cuda")
    kc = torch.zeros((cfg.kv_heads, cfg.ctx_max, cfg.head_dim), device="cuda")
    vc = torch.zeros_like(kc)
    table = torch.empty(cfg.head_dim, device="cuda")
    kernels.rope_table_dev(dec.pos, cfg.rope_theta, cfg.head_dim, table)
    L.wqkv.matmul_qkv_rope(dec.h, q, kc, vc, cfg.heads, cfg.kv_heads, cfg.head_dim, cfg.ctx_max, dec.pos, cfg.rope_theta,
                           gain=L.attn_norm, eps=cfg.rms_eps, rope_table=table)
    kernels.sync()
    src = f"l{layer % 4}"
    xn = rms(h, w.host[f"{src}.attn_norm"], cfg.rms_eps)
    n = cfg.q_dim + 2 * cfg.kv_dim
    qkv = packed_rows(w.host, f"{src}.wqkv", cfg.linear_encoding, cfg.hidden, np.arange(n)) @ xn

    def rope(x):                                    # [heads, head_dim], adjacent pairs, float64
        ang = pos * cfg.rope_theta ** (-2.0 * np.arange(cfg.head_dim // 2) / cfg.head_dim)
        out = np.empty_like(x)
        out[:, 0::2] = x[:, 0::2] * np.cos(ang) - x[:, 1::2] * np.sin(ang)
        out[:, 1::2] = x[:, 0::2] * np.sin(ang) + x[:, 1::2] * np.cos(ang)
        return out

    q_ref = rope(qkv[:cfg.q_dim].reshape(cfg.heads, cfg.head_dim))
    k_ref = rope(qkv[cfg.q_dim:cfg.q_dim + cfg.kv_dim].reshape(cfg.kv_heads, cfg.head_dim))
    v_ref = qkv[cfg.q_dim + cfg.kv_dim:].reshape(cfg.kv_heads, cfg.head_dim)
    scale = np.abs(qkv).max()
    assert np.abs(q.cpu().numpy().reshape(cfg.heads, cfg.head_dim) - q_ref).max() <= 1e-3 * scale
    kh, vh = kc.cpu().numpy(), vc.cpu().numpy()
    assert np.abs(kh[:, pos] - k_ref).max() <= 1e-3 * scale
    assert np.abs(vh[:, pos] - v_ref).max() <= 1e-3 * scale
    kh[:, pos] = 0
    vh[:, pos] = 0
    assert not kh.any() and not vh.any()           # only row `pos` of every kv head was written


def test_attention_over_more_than_1024_cached_keys(full_stack):
    """The last layer's single-query attention of the last step: its query, cache rows and output are still on the device."""
    cfg, w, dec, *_ = full_stack
    n_keys = dec.position()                         # the step consumed the token at position n_keys - 1
    assert n_keys > 1024
    li = cfg.layers - 1
    q = dec.q.download(np.float32, cfg.q_dim).reshape(cfg.heads, cfg.head_dim).astype(np.float64)
    out = dec.attn.download(np.float32, cfg.q_dim).reshape(cfg.heads, cfg.head_dim)
    k = dec.k_cache.download(np.float32, dec.kv_layer_floats, 4 * li * dec.kv_layer_floats).reshape(cfg.kv_heads, cfg.ctx_max, cfg.head_dim)
    v = dec.v_cache.download(np.float32, dec.kv_layer_floats, 4 * li * dec.kv_layer_floats).reshape(cfg.kv_heads, cfg.ctx_max, cfg.head_dim)
    per = cfg.heads // cfg.kv_heads
    want = np.empty_like(q)
    for hh in range(cfg.heads):
        kk, vv = k[hh // per, :n_keys].astype(np.float64), v[hh // per, :n_keys].astype(np.float64)
        s = kk @ q[hh] / np.sqrt(cfg.head_dim)
        p = np.exp(s - s.max())
        want[hh] = (p / p.sum()) @ vv
    assert max_norm_err(out, want) < 1e-4


def test_two_layers_at_full_widths_teacher_forced_against_float64():
    """Hidden 4096, FFN 14336, 32 / 8 heads of 128 (vocabulary 32064 to keep the float64 checker small): prefill through
    the fp32 route (6 tokens) and the MFMA route (24 tokens), then greedy decode steps, logits against the checker at
    every step."""
    from dataclasses import replace
    from skainet_amd.decoder import LLAMA3_8B, LlamaDecoder, LlamaWeights
    cfg = replace(LLAMA3_8B, layers=2, vocab=32064, ctx_max=64)
    w = LlamaWeights(cfg, seed=99, keep_host=True)
    chk_weights = CheckDecoder(cfg, w.host)
    for prompt_len, tol in ((6, 1e-3), (24, 2e-2)):
        chk = CheckDecoder.__new__(CheckDecoder)
        chk.__dict__.update(chk_weights.__dict__)
        chk.k = [np.zeros((cfg.kv_heads, 0, cfg.head_dim)) for _ in range(cfg.layers)]
        chk.v = [np.zeros((cfg.kv_heads, 0, cfg.head_dim)) for _ in range(cfg.layers)]
        prompt = np.random.default_rng(prompt_len).integers(0, cfg.vocab, prompt_len)
        dec = LlamaDecoder(w, max_prefill=32)
        tok = dec.prefill(prompt)
        h_ref, logits_ref = chk.forward(prompt)
        assert max_norm_err(dec.hidden_rows(prompt_len), h_ref) < tol
        assert max_norm_err(dec.last_logits(), logits_ref) < tol
        if prompt_len == 6:
            for i in range(6):
                top2 = np.sort(logits_ref)[-2:]
                if top2[1] - top2[0] > 2e-3 * np.abs(logits_ref).max():
                    assert tok == int(np.argmax(logits_ref)), f"step {i}"
                _, logits_ref = chk.forward([tok])
                tok = int(dec.decode(1, use_graph=(i % 2 == 1))[0])
                assert max_norm_err(dec.last_logits(), logits_ref) < 1e-3, f"step {i}"
                assert tok == int(np.argmax(dec.last_logits()))
        dec.close()
