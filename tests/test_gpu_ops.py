"""The generic resident-activation ops class (skainet_amd/ops.py, the host-side mirror of a HipOps : DefaultCpuOpsBase
after WasmCpuOps.kt:180-428) against closed forms in float64, and a Llama stack written against that class alone against
the decoder's float64 checker (tests/decoder_check.py) and against the fused decoder.

Tolerances: elementwise arithmetic bit-exact, activations / norms / softmax 2e-6 .. 1e-5 of the largest value, dense
products 1e-5, attention 1e-4 (the reference's own assertClose); the stack 1e-3 on the fp32 routes (decode, prompts of at
most 8 tokens) and 2e-2 through the bf16 MFMA prefill."""
import math

import numpy as np
import pytest

from decoder_check import CheckDecoder
from gpu_util import gaussian_weight
from oracle import lib as L

pytestmark = pytest.mark.gpu


def max_norm_err(got, ref):
    ref = np.asarray(ref, np.float64)
    return float(np.abs(np.asarray(got, np.float64) - ref).max() / max(np.abs(ref).max(), 1e-30))


@pytest.fixture(scope="module")
def ops(hip_backend):
    from skainet_amd.ops import ForwardScope, HipOps
    scope = ForwardScope(64 << 20)
    yield HipOps(scope)
    scope.close()


def test_elementwise_activations_and_reductions_stay_resident(ops):
    rng = np.random.default_rng(1)
    a, b = rng.standard_normal((7, 33)).astype(np.float32), rng.standard_normal((7, 33)).astype(np.float32) + 3.0
    bias, one = rng.standard_normal((1, 33)).astype(np.float32), np.array([1.5], np.float32)
    A, B, BIAS, ONE = (ops.to_resident(t) for t in (a, b, bias, one))
    for name, fn in (("add", np.add), ("subtract", np.subtract), ("multiply", np.multiply), ("divide", np.divide)):
        for (x, X), (y, Y) in (((a, A), (b, B)), ((a, A), (bias, BIAS)), ((one, ONE), (b, B))):
            got = getattr(ops, name)(X, Y)
            assert got.shape == np.broadcast_shapes(x.shape, y.shape)
            assert np.array_equal(got.numpy(), fn(x, y)), name                     # one IEEE operation per element
    with pytest.raises(ValueError):
        ops.add(A, ops.to_resident(np.zeros((7, 1), np.float32)))                   # a column broadcast is none of the three modes
    x64 = a.astype(np.float64)
    erf = np.vectorize(math.erf)
    for name, ref in (("relu", np.maximum(x64, 0)), ("sigmoid", 1 / (1 + np.exp(-x64))), ("silu", x64 / (1 + np.exp(-x64))),
                      ("tanh", np.tanh(x64)), ("erf", erf(x64)), ("gelu", 0.5 * x64 * (1 + erf(x64 / np.sqrt(2))))):
        assert max_norm_err(getattr(ops, name)(A).numpy(), ref) <= 2e-6, name
    tanh_gelu = 0.5 * x64 * (1 + np.tanh(np.sqrt(2 / np.pi) * (x64 + 0.044715 * x64 ** 3)))
    assert max_norm_err(ops.gelu(A, approximate=True).numpy(), tanh_gelu) <= 2e-6
    t = rng.standard_normal((3, 5, 8)).astype(np.float32)
    T = ops.to_resident(t)
    assert abs(float(ops.sum(T).numpy()) - t.astype(np.float64).sum()) <= 1e-5 * np.abs(t).sum()
    assert abs(float(ops.mean(T).numpy()) - t.astype(np.float64).mean()) <= 1e-6
    for dim in (0, 1, 2, -1):
        assert max_norm_err(ops.sum(T, dim).numpy(), t.astype(np.float64).sum(axis=dim)) <= 2e-6
        assert max_norm_err(ops.mean(T, dim).numpy(), t.astype(np.float64).mean(axis=dim)) <= 2e-6
    ops.scope.reset()


def test_a_tensor_of_a_forward_scope_is_dead_after_the_reset(hip_backend):
    """Per-step activations belong to their scope (Scope.kt:206-215: reset closes what was handed out, a later use
    throws): a tensor, its views, and an op on it all raise after the reset; a tensor made after the reset lives at the
    address the first one had; a tensor without a scope is not touched by any of it."""
    from skainet_amd._lib import HipError
    from skainet_amd.ops import ForwardScope, HipOps
    scope = ForwardScope(1 << 20)
    try:
        o, free = HipOps(scope), HipOps()
        keep = free.to_resident(np.arange(6, dtype=np.float32).reshape(2, 3))
        t = o.to_resident(np.ones((4, 8), np.float32))
        view = t.rows(1, 2).reshape(16)
        first = t.ptr
        assert o.add(t, t).numpy().sum() == 64.0
        scope.reset()
        for stale in (t, view):
            with pytest.raises(HipError):
                stale.numpy()
        with pytest.raises(HipError):
            o.relu(t)
        again = o.to_resident(np.zeros((4, 8), np.float32))
        assert again.ptr == first and again.numpy().sum() == 0.0
        assert keep.numpy().tolist() == [[0.0, 1.0, 2.0], [3.0, 4.0, 5.0]]
        with pytest.raises(HipError):
            o.empty((1 << 20,))                                        # 4 MB out of a 1 MB slab
    finally:
        scope.close()
    with pytest.raises(HipError):
        again.numpy()                                                  # the scope is gone


def test_softmax_norms_matmuls_and_attention(ops, hip_backend):
    rng = np.random.default_rng(2)
    x = rng.standard_normal((6, 50)).astype(np.float32) * 3
    X = ops.to_resident(x)
    e = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
    sm = e / e.sum(axis=1, keepdims=True)
    assert max_norm_err(ops.softmax(X).numpy(), sm) <= 2e-6
    assert max_norm_err(ops.log_softmax(X, -1).numpy(), np.log(sm)) <= 2e-6
    with pytest.raises(ValueError):
        ops.softmax(X, 0)
    g, bta = rng.standard_normal(50).astype(np.float32), rng.standard_normal(50).astype(np.float32)
    G, Bt = ops.to_resident(g), ops.to_resident(bta)
    x64 = x.astype(np.float64)
    rms = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-5) * g
    assert max_norm_err(ops.rms_norm(X, G, 1e-5).numpy(), rms) <= 1e-5
    mu, var = x64.mean(axis=1, keepdims=True), x64.var(axis=1, keepdims=True)
    assert max_norm_err(ops.layer_norm(X, G, Bt, 1e-5).numpy(), (x64 - mu) / np.sqrt(var + 1e-5) * g + bta) <= 1e-5
    # dense products: A . B and x . W^T, outputs resident and fed on
    a, b = rng.standard_normal((9, 40)).astype(np.float32), rng.standard_normal((40, 21)).astype(np.float32)
    C = ops.matmul(ops.to_resident(a), ops.to_resident(b))
    assert max_norm_err(C.numpy(), a.astype(np.float64) @ b.astype(np.float64)) <= 1e-5
    w = rng.standard_normal((13, 21)).astype(np.float32)
    D = ops.matmul_weight_transposed(C, ops.to_resident(w))
    assert D.shape == (9, 13)
    assert max_norm_err(D.numpy(), (a.astype(np.float64) @ b.astype(np.float64)) @ w.astype(np.float64).T) <= 2e-5
    with pytest.raises(ValueError):
        ops.matmul(ops.to_resident(a), ops.to_resident(w))
    # a packed weight takes the product its view kernel runs (one row: the matrix-core GEMV; many rows: the MFMA GEMM)
    n, k = 96, 1024
    packed = gaussian_weight(hip_backend, "Q4_K", n, k, 5)
    W = hip_backend.DeviceWeight.upload("Q4_K", packed, n, k)
    for m, tol in ((1, 1e-3), (3, 1e-3), (24, 2e-2)):
        xs = rng.standard_normal((m, k)).astype(np.float32)
        got = ops.matmul_weight_transposed(ops.to_resident(xs), W)
        assert got.shape == (m, n) and max_norm_err(got.numpy(), L.gemv("Q4_K", xs, packed, n)) <= tol
    # attention: GQA, causal, against the oracle's restatement of the reference's fused kernel
    q = rng.standard_normal((2, 8, 5, 64)).astype(np.float32)
    kk, vv = rng.standard_normal((2, 2, 5, 64)).astype(np.float32), rng.standard_normal((2, 2, 5, 64)).astype(np.float32)
    out = ops.scaled_dot_product_attention(ops.to_resident(q), ops.to_resident(kk), ops.to_resident(vv), causal=True)
    assert np.abs(out.numpy() - L.sdpa(q, kk, vv, 0.125, True)).max() <= 1e-4
    ops.scope.reset()


def small_config():
    from skainet_amd.decoder import LlamaConfig
    return LlamaConfig(layers=3, hidden=512, heads=8, kv_heads=2, head_dim=64, ffn=1024, vocab=1024, ctx_max=64, rope_theta=10000.0)


@pytest.mark.parametrize("prompt_len,tol", [(5, 1e-3), (24, 2e-2)])
def test_llama_stack_through_the_generic_ops_matches_the_checker_and_the_fused_decoder(hip_backend, prompt_len, tol):
    """Prefill and greedy decode through HipOps alone (one device entry per op, nothing fused by name): logits against the
    float64 checker after the prompt and after every decode step, tokens against the fused decoder's, and the recorded
    graph of a step (the forward scopes hand out the same addresses every step) against eager steps."""
    from skainet_amd.decoder import LlamaDecoder, LlamaWeights
    from skainet_amd.ops_decoder import OpsLlamaDecoder, OpsLlamaWeights
    cfg = small_config()
    w = LlamaWeights(cfg, seed=21, sigma=0.05, keep_host=True)
    ow = OpsLlamaWeights(w)
    prompt = np.random.default_rng(77).integers(0, cfg.vocab, prompt_len)
    chk = CheckDecoder(cfg, w.host)
    _, logits_ref = chk.forward(prompt)
    fused = LlamaDecoder(w, max_prefill=32)
    first_fused = fused.prefill(prompt)
    outs = []
    for use_graph in (False, True):
        dec = OpsLlamaDecoder(ow, max_prefill=32)
        tok = dec.prefill(prompt)
        assert max_norm_err(dec.last_logits(), logits_ref) < tol
        toks = [tok]
        if not use_graph:
            ref = logits_ref
            for i in range(6):
                _, ref = chk.forward([tok])
                tok = int(dec.decode(1, use_graph=False)[0])
                assert max_norm_err(dec.last_logits(), ref) < tol, f"step {i}"
                assert dec.position() == prompt_len + i + 1
                toks.append(tok)
            chk = None
        else:
            toks += [int(t) for t in dec.decode(6, use_graph=True)]
        outs.append((toks, dec.last_logits()))
        dec.close()
    assert outs[0][0] == outs[1][0]                                  # graph replays = eager steps
    assert np.array_equal(outs[0][1], outs[1][1])
    if tol == 1e-3:
        assert outs[0][0][0] == first_fused
        assert outs[0][0][1:] == [int(t) for t in fused.decode(6, use_graph=False)]
    assert OpsLlamaDecoder.launches_per_token(type("D", (), {"cfg": cfg})()) == 17 * cfg.layers + 5
