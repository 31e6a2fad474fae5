"""GPU parity: fused row kernels, attention and dense matmuls against the oracle (and the reference C library's
recorded vectors). Tolerances: the reference's own for fused rows (rel 1e-4, abs 1e-5, NativeFusedKernelsTest.kt:166-218);
2e-2 normalised is the task's bound for attention, the fp32 kernels here are held to 1e-4.
"""
import os

import numpy as np
import pytest

from oracle import lib as L
from gpu_util import dev, normalized_err
from test_oracle_golden import SDPA_GRID, fill, sdpa_fp64, sdpa_inputs

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def close(got, want, rel=1e-4, abs_=1e-5):
    """assertClose of NativeFusedKernelsTest.kt:53-61: |d| <= max|want| * rel + abs."""
    tol = np.abs(want).max() * rel + abs_
    d = np.abs(np.asarray(got, np.float64) - want).max()
    assert d <= tol, (d, tol)


def gpu_sdpa(kernels, torch, q, k, v, scale, causal=False, window=0, rc=0, lengths=None, mask=None):
    b, h, sq, d = q.shape
    hkv, skv = k.shape[1], k.shape[2]
    out = torch.full(q.shape, float("nan"), dtype=torch.float32, device="cuda")
    md = (0, 0, 0, 0)
    dm = None
    if mask is not None:
        md = tuple([1] * (4 - mask.ndim) + list(mask.shape))
        dm = dev(torch, mask)
    dl = None if lengths is None else dev(torch, np.asarray(lengths, np.int32))
    kernels.sdpa_dev(dev(torch, q), dev(torch, k), dev(torch, v), out, b, h, hkv, sq, skv, d, scale, causal, window, rc, dl, dm, md)
    return out.cpu().numpy()


@pytest.mark.parametrize("case", SDPA_GRID)
def test_attention_every_mask_rule(hip_backend, torch_cuda, case):
    h, hkv, sq, skv, causal, use_len, win, rc = case
    q, k, v = sdpa_inputs(3, h, hkv, sq, skv, 8)
    lengths = np.array([skv, (skv + 1) // 2, 1], np.int32) if use_len else None
    scale = float(1.0 / np.sqrt(8))
    got = gpu_sdpa(hip_backend, torch_cuda, q, k, v, scale, causal, win, rc, lengths)
    close(got, L.sdpa(q, k, v, scale, causal, win, rc, lengths))
    recorded = np.load(os.path.join(HERE, "golden", "ref_vectors.npz"))[f"sdpa/{SDPA_GRID.index(case)}"]
    close(got, recorded)
    # the structured rules equal the dense -1e30 mask (AttentionMask.additive)
    dense = np.full((3, 1, sq, skv), -1e30, np.float32)
    for b in range(3):
        for qi in range(sq):
            absq = skv - sq + qi
            first = max(0, absq - win + 1) if win > 0 else 0
            end = min(skv, lengths[b] if use_len else skv)
            if causal:
                end = min(end, absq + 1)
            if win > 0:
                end = min(end, absq + rc + 1)
            dense[b, 0, qi, first:max(end, first)] = 0.0
    close(gpu_sdpa(hip_backend, torch_cuda, q, k, v, scale, mask=dense), got, rel=1e-5, abs_=1e-6)


def test_attention_masks_padding_and_host_entry(hip_backend, torch_cuda):
    q, k, v = sdpa_inputs(2, 4, 2, 5, 9, 16, seed=4)
    for mask in (fill(9, 6).reshape(1, 1, 1, 9), fill(45, 7).reshape(5, 9), fill(2 * 4 * 5 * 9, 8).reshape(2, 4, 5, 9),
                 fill(2 * 2 * 5 * 9, 9).reshape(2, 2, 5, 9)):
        close(gpu_sdpa(hip_backend, torch_cuda, q, k, v, 0.3, True, mask=mask), L.sdpa(q, k, v, 0.3, True, mask=mask))
    q, k, v = sdpa_inputs(2, 2, 2, 3, 5, 4)
    out = gpu_sdpa(hip_backend, torch_cuda, q, k, v, 0.5, lengths=[0, 5])
    assert np.isfinite(out).all()
    close(out, L.sdpa(q, k, v, 0.5, lengths=np.array([0, 5], np.int32)), rel=1e-5, abs_=1e-6)
    # seq_kv == 0 zeroes the output; the SPI kernel on host arrays goes through the same path
    attn = hip_backend.HipKernelProvider().attention_fp32()
    o = np.full(q.shape, 5, np.float32)
    attn.sdpa(q, k[:, :, :0].copy(), v[:, :, :0].copy(), o, 2, 2, 2, 3, 0, 4, 0.5, False, 0, 0)
    assert not o.any()
    q, k, v = sdpa_inputs(1, 12, 12, 150, 150, 64, seed=9)     # the reference's threaded shape (NativeFusedKernelsTest.kt:211)
    o = np.empty_like(q)
    want = L.sdpa(q, k, v, 1 / np.sqrt(64.0), True)
    attn.sdpa(q, k, v, o, 1, 12, 12, 150, 150, 64, float(1 / np.sqrt(64.0)), True, 0, 0)
    assert normalized_err(o, want, eps=1.0) <= 2e-2               # a prompt shape: bf16 operands on the matrix cores
    hip_backend.set_tuning("sdpa_prefill_mfma", 0)                # the same call on the fp32 kernel: the reference's tolerance
    try:
        attn.sdpa(q, k, v, o, 1, 12, 12, 150, 150, 64, float(1 / np.sqrt(64.0)), True, 0, 0)
    finally:
        hip_backend.set_tuning("sdpa_prefill_mfma", 1)
    close(o, want)
    with pytest.raises(ValueError):
        attn.sdpa(q, k, v, o, 1, 12, 12, 150, 150, 64, 0.1, True, 0, 2)


@pytest.mark.parametrize("batch", [1, 8])
def test_attention_decode_config(hip_backend, torch_cuda, batch):
    """Decode: one query token against a KV cache of 4096, 32 query / 8 KV heads, head_dim 128."""
    rng = np.random.default_rng(50 + batch)
    q = rng.standard_normal((batch, 32, 1, 128)).astype(np.float32)
    k = rng.standard_normal((batch, 8, 4096, 128)).astype(np.float32)
    v = rng.standard_normal((batch, 8, 4096, 128)).astype(np.float32)
    scale = float(1 / np.sqrt(128.0))
    got = gpu_sdpa(hip_backend, torch_cuda, q, k, v, scale, True)
    want = L.sdpa(q, k, v, scale, True)
    err = normalized_err(got, want)
    print(f"decode attention batch {batch}: normalized max err {err:.2e}")
    assert err <= 2e-2
    lengths = np.arange(1, batch + 1, dtype=np.int32) * 500
    close(gpu_sdpa(hip_backend, torch_cuda, q, k, v, scale, True, 1024, 0, lengths), L.sdpa(q, k, v, scale, True, 1024, 0, lengths))


@pytest.mark.parametrize("heads,kv_heads,d,skv,batch", [(8, 2, 64, 700, 2), (4, 4, 128, 33, 3), (16, 2, 128, 1500, 1),
                                                         (6, 3, 256, 260, 2), (2, 1, 64, 16, 1), (32, 8, 128, 2048, 1),
                                                         (12, 4, 64, 5000, 1), (5, 5, 96, 300, 2)])
def test_attention_decode_kernel_shapes_and_rules(hip_backend, torch_cuda, heads, kv_heads, d, skv, batch):
    """The one-query kernel over its head shapes (group sizes 1 / 2 / 4 / 8-as-2x4, head_dim 64 / 128 / 256; 96 stays
    on the general kernel), split and unsplit key ranges, key lengths (one of them 0: uniform weights), windows,
    and twice in a row so the split counters are known to come back to zero."""
    rng = np.random.default_rng(heads * d + skv)
    q = rng.standard_normal((batch, heads, 1, d)).astype(np.float32)
    k = rng.standard_normal((batch, kv_heads, skv, d)).astype(np.float32)
    v = rng.standard_normal((batch, kv_heads, skv, d)).astype(np.float32)
    scale = float(1 / np.sqrt(d))
    lengths = np.array([skv, 0, skv // 3][:batch], np.int32)
    for causal, win, rc, lens in ((True, 0, 0, None), (False, 0, 0, lengths), (True, max(1, skv // 5), 0, None),
                                  (True, max(2, skv // 2), 1, lengths), (True, 0, 0, None)):
        got = gpu_sdpa(hip_backend, torch_cuda, q, k, v, scale, causal, win, rc, lens)
        close(got, L.sdpa(q, k, v, scale, causal, win, rc, lens), rel=2e-5, abs_=2e-6)


def test_attention_prefill_config_against_torch_fp32(hip_backend, torch_cuda):
    """Prefill: seq 2048 causal, 32 / 8 heads, head_dim 128. The oracle checks a 256-long prefix problem exactly;
    the full size is compared with torch's fp32 attention on the same device (textbook softmax(QK^T)V)."""
    torch = torch_cuda
    rng = np.random.default_rng(60)
    s = 2048
    q = rng.standard_normal((1, 32, s, 128)).astype(np.float32)
    k = rng.standard_normal((1, 8, s, 128)).astype(np.float32)
    v = rng.standard_normal((1, 8, s, 128)).astype(np.float32)
    scale = float(1 / np.sqrt(128.0))
    got = gpu_sdpa(hip_backend, torch, q, k, v, scale, True)
    tq, tk, tv = dev(torch, q), dev(torch, k).repeat_interleave(4, 1), dev(torch, v).repeat_interleave(4, 1)
    sc = torch.matmul(tq, tk.transpose(-1, -2)) * scale
    sc = sc.masked_fill(~torch.ones(s, s, dtype=torch.bool, device="cuda").tril(), -1e30)
    want = torch.matmul(torch.softmax(sc, -1), tv).cpu().numpy()
    # bf16 operands: the bound is on the error against the largest output magnitude (per-element relative error of a
    # near-zero output is unbounded for any reordered or reduced-precision sum), plus an RMS bound
    err = normalized_err(got, want, eps=1.0)
    rms = float(np.sqrt(np.mean((got - want) ** 2)) / np.abs(want).max())
    print(f"prefill attention 2048: max err / max |ref| vs torch fp32 {err:.2e}, rms {rms:.2e}")
    assert err <= 2e-2 and rms <= 5e-3
    sp = 256
    qs, ks, vs = q[:, :, :sp].copy(), k[:, :, :sp].copy(), v[:, :, :sp].copy()
    want_s = L.sdpa(qs, ks, vs, scale, True)
    e_mfma = normalized_err(gpu_sdpa(hip_backend, torch, qs, ks, vs, scale, True), want_s, eps=1.0)
    print(f"prefill attention 256 (matrix cores): max err / max |ref| vs oracle {e_mfma:.2e}")
    assert e_mfma <= 2e-2
    hip_backend.set_tuning("sdpa_prefill_mfma", 0)                # the fp32 kernel on the same problem, reference tolerance
    try:
        close(gpu_sdpa(hip_backend, torch, qs, ks, vs, scale, True), want_s)
    finally:
        hip_backend.set_tuning("sdpa_prefill_mfma", 1)
    # causal prefix property: the first 256 rows of the long problem are the short problem
    assert normalized_err(got[:, :, :sp], want_s, eps=1.0) <= 2e-2


@pytest.mark.parametrize("batch,heads,kv_heads,d,sq,skv,causal", [
    (1, 8, 2, 128, 200, 200, True), (2, 4, 4, 64, 97, 97, True), (1, 6, 3, 128, 64, 333, True), (1, 16, 2, 64, 130, 130, False),
    (1, 2, 1, 128, 31, 1000, True), (2, 8, 8, 64, 512, 512, True), (1, 4, 1, 128, 16, 16, True), (1, 3, 3, 128, 100, 257, False)])
def test_attention_prefill_mfma_shapes(hip_backend, torch_cuda, batch, heads, kv_heads, d, sq, skv, causal):
    """The matrix-core prompt kernel over its shape range: group sizes 1 / 2 / 4 / 8, head_dim 64 / 128, lengths that
    are not multiples of the 32-query or 64-key tiles, a query block shorter than the keys (a later prompt chunk),
    causal and full. Bound: 2e-2 of the largest reference magnitude (bf16 operands); the RMS error is held to 5e-3."""
    rng = np.random.default_rng(sq * skv + d)
    q = rng.standard_normal((batch, heads, sq, d)).astype(np.float32)
    k = rng.standard_normal((batch, kv_heads, skv, d)).astype(np.float32)
    v = rng.standard_normal((batch, kv_heads, skv, d)).astype(np.float32)
    scale = float(1 / np.sqrt(d))
    got = gpu_sdpa(hip_backend, torch_cuda, q, k, v, scale, causal)
    want = L.sdpa(q, k, v, scale, causal)
    assert np.isfinite(got).all()
    assert normalized_err(got, want, eps=1.0) <= 2e-2
    assert np.sqrt(np.mean((got - want) ** 2)) <= 5e-3 * np.abs(want).max()
    # rows of P sum to 1: with v = 1 everywhere the output is 1 (bf16 P entries: 1e-2)
    ones = np.ones_like(v)
    assert np.abs(gpu_sdpa(hip_backend, torch_cuda, q, k, ones, scale, causal) - 1.0).max() <= 1e-2


@pytest.mark.parametrize("batch,heads,kv_heads,d,sq,skv,causal,window,rc,lengths", [
    (1, 8, 2, 128, 300, 300, True, 64, 0, None),            # sliding window shorter than a key block ... 
    (1, 8, 2, 128, 300, 300, True, 100, 0, None),           # ... and one that straddles blocks
    (2, 4, 2, 64, 200, 200, True, 0, 0, [200, 77]),         # key lengths: the second sequence ends inside a block
    (3, 4, 4, 64, 130, 130, True, 50, 0, [130, 40, 0]),     # window + lengths: late queries of sequence 1 and all of 2 keep no key
    (1, 4, 1, 128, 96, 400, True, 128, 0, None),            # a later prompt chunk with a window
    (1, 6, 3, 128, 150, 150, False, 40, 7, None),           # bidirectional window with right context
    (2, 2, 2, 64, 64, 64, False, 0, 0, [1, 64]),            # full attention, one key
    (1, 32, 8, 128, 512, 512, True, 256, 0, None),          # the Llama-3 head shape with a 256-key window
])
def test_attention_prefill_mfma_window_and_key_lengths(hip_backend, torch_cuda, batch, heads, kv_heads, d, sq, skv, causal, window,
                                                       rc, lengths):
    """The matrix-core prompt kernel under the structured rules (sliding window, right context, per-sequence key
    lengths), including queries the rules leave without a key (equal weight on every key, as the reference's row of
    equal -1e30 scores). Against the oracle, 2e-2 of the largest reference magnitude; the fp32 kernel on the same call
    stays within the reference's own tolerance."""
    rng = np.random.default_rng(sq * skv + d + window)
    q = rng.standard_normal((batch, heads, sq, d)).astype(np.float32)
    k = rng.standard_normal((batch, kv_heads, skv, d)).astype(np.float32)
    v = rng.standard_normal((batch, kv_heads, skv, d)).astype(np.float32)
    scale = float(1 / np.sqrt(d))
    ln = None if lengths is None else np.asarray(lengths, np.int32)
    want = L.sdpa(q, k, v, scale, causal, window, rc, ln)
    try:
        for teams in (1, 2):        # one query group per workgroup; a late and an early (or two neighbouring) groups paired
            hip_backend.set_tuning("sdpa_prefill_teams", teams)
            got = gpu_sdpa(hip_backend, torch_cuda, q, k, v, scale, causal, window, rc, ln)
            assert hip_backend.last_kernel() == "sdpa_prefill_kernel"
            assert np.isfinite(got).all()
            assert normalized_err(got, want, eps=1.0) <= 2e-2
            assert np.sqrt(np.mean((got - want) ** 2)) <= 5e-3 * np.abs(want).max()
    finally:
        hip_backend.set_tuning("sdpa_prefill_teams", 0)
    ones = np.ones_like(v)
    assert np.abs(gpu_sdpa(hip_backend, torch_cuda, q, k, ones, scale, causal, window, rc, ln) - 1.0).max() <= 1e-2
    hip_backend.set_tuning("sdpa_prefill_mfma", 0)
    try:
        close(gpu_sdpa(hip_backend, torch_cuda, q, k, v, scale, causal, window, rc, ln), want)
        assert hip_backend.last_kernel() != "sdpa_prefill_kernel"
    finally:
        hip_backend.set_tuning("sdpa_prefill_mfma", 1)


@pytest.mark.parametrize("batch,heads,kv_heads,d,sq,skv,causal,window,lengths,mask_dims", [
    (2, 8, 2, 64, 200, 200, True, 0, None, (1, 1, 200, 200)),        # one bias matrix for every head (ALiBi-like), causal
    (2, 8, 2, 128, 96, 160, False, 0, [160, 70], (2, 8, 96, 160)),   # a bias per batch and head, ragged key lengths, a prompt chunk
    (1, 4, 4, 64, 130, 132, True, 48, None, (1, 4, 1, 132)),         # per-head key bias broadcast over queries, window (late queries lose keys)
    (3, 6, 3, 128, 64, 64, True, 0, [64, 10, 0], (3, 3, 64, 64)),    # a bias per KV head; sequence 2 has no key at all
    (2, 4, 2, 64, 80, 80, False, 0, None, (2, 1, 80, 1)),            # one value per query row: shifts every score of the row alike
    (1, 32, 8, 128, 512, 512, True, 0, None, (1, 1, 512, 512)),      # the Llama-3 head shape with a padding-style mask of -1e9 entries
])
def test_attention_prefill_mfma_with_an_additive_mask(hip_backend, torch_cuda, batch, heads, kv_heads, d, sq, skv, causal, window,
                                                      lengths, mask_dims):
    """The matrix-core prompt kernel with an additive mask in every broadcast form the reference accepts, alone and on
    top of the structured rules: the mask is added to every score, an excluded key's -1e30 included, so a row the rules
    leave without a key weighs the keys by its mask values' softmax only if those differ by less than fp32 resolves at
    1e30 -- i.e. equally. Against the oracle, 2e-2 of the largest reference magnitude; masks whose rows are not a
    multiple of four keys stay on the fp32 kernel."""
    rng = np.random.default_rng(sq * skv + d + mask_dims[0])
    q = rng.standard_normal((batch, heads, sq, d)).astype(np.float32)
    k = rng.standard_normal((batch, kv_heads, skv, d)).astype(np.float32)
    v = rng.standard_normal((batch, kv_heads, skv, d)).astype(np.float32)
    scale = float(1 / np.sqrt(d))
    mask = (rng.standard_normal(mask_dims) * 2).astype(np.float32)
    if mask_dims[3] > 1:
        mask[..., rng.random(mask_dims[3]) < 0.2] = -1e9              # some keys switched off for everyone, as a padding mask does
        mask[..., 0] = np.minimum(mask[..., 0], 3.0)                   # and key 0 stays available
        mask[..., 0] = np.maximum(mask[..., 0], -3.0)
    ln = None if lengths is None else np.asarray(lengths, np.int32)
    want = L.sdpa(q, k, v, scale, causal, window, 0, ln, mask)
    try:
        for teams in (1, 2):
            hip_backend.set_tuning("sdpa_prefill_teams", teams)
            got = gpu_sdpa(hip_backend, torch_cuda, q, k, v, scale, causal, window, 0, ln, mask)
            assert hip_backend.last_kernel() == "sdpa_prefill_kernel"
            assert np.isfinite(got).all()
            assert normalized_err(got, want, eps=1.0) <= 2e-2
            assert np.sqrt(np.mean((got - want) ** 2)) <= 5e-3 * np.abs(want).max()
    finally:
        hip_backend.set_tuning("sdpa_prefill_teams", 0)
    hip_backend.set_tuning("sdpa_prefill_mfma", 0)
    try:
        close(gpu_sdpa(hip_backend, torch_cuda, q, k, v, scale, causal, window, 0, ln, mask), want)
        assert hip_backend.last_kernel() != "sdpa_prefill_kernel"
    finally:
        hip_backend.set_tuning("sdpa_prefill_mfma", 1)
    if mask_dims[3] > 4:
        odd = np.ascontiguousarray(mask[..., : mask_dims[3] - 1])     # rows of skv - 1 keys: not the layout the kernel reads
        got_odd = gpu_sdpa(hip_backend, torch_cuda, q, k[:, :, : skv - 1], v[:, :, : skv - 1], scale, causal, window, 0,
                           None if ln is None else np.minimum(ln, skv - 1), odd) if sq <= skv - 1 else None
        if got_odd is not None:
            assert hip_backend.last_kernel() != "sdpa_prefill_kernel" or (skv - 1) % 4 == 0
            close(got_odd, L.sdpa(q, k[:, :, : skv - 1], v[:, :, : skv - 1], scale, causal, window, 0,
                                  None if ln is None else np.minimum(ln, skv - 1), odd))


def test_norms_softmax_and_glue(hip_backend, torch_cuda):
    torch = torch_cuda
    kx = hip_backend
    rows, cols = 5, 4096
    x = (np.random.default_rng(1).standard_normal((rows, cols)) * 3).astype(np.float32)
    g = np.random.default_rng(2).standard_normal(cols).astype(np.float32)
    bta = np.random.default_rng(3).standard_normal(cols).astype(np.float32)
    xd = x.astype(np.float64)
    out = torch.empty(rows, cols, device="cuda")
    kx.rms_norm_dev(dev(torch, x), dev(torch, g), out, rows, cols, 1e-5)
    close(out.cpu().numpy(), xd / np.sqrt((xd * xd).mean(1, keepdims=True) + 1e-5) * g, abs_=1e-4)
    ref = np.empty_like(x)
    L.oracle().orc_f32_rms_norm(L.fp(x), L.fp(g), L.fp(ref), rows, cols, 1e-5)
    close(out.cpu().numpy(), ref, rel=1e-5)
    kx.rms_norm_dev(dev(torch, x), None, out, rows, cols, 1e-5)
    close(out.cpu().numpy(), xd / np.sqrt((xd * xd).mean(1, keepdims=True) + 1e-5), abs_=1e-4)
    kx.layer_norm_dev(dev(torch, x), dev(torch, g), dev(torch, bta), out, rows, cols, 1e-5)
    mu, var = xd.mean(1, keepdims=True), xd.var(1, keepdims=True)
    close(out.cpu().numpy(), (xd - mu) / np.sqrt(var + 1e-5) * g + bta, abs_=1e-4)
    for log in (False, True):
        kx.softmax_rows_dev(dev(torch, x), out, rows, cols, log)
        want = np.empty_like(x)
        L.oracle().orc_f32_softmax_rows(L.fp(x), L.fp(want), rows, cols, int(log))
        close(out.cpu().numpy(), want, rel=1e-5, abs_=1e-6)
    n = 14336 * 3 + 5
    a = np.random.default_rng(4).standard_normal(n).astype(np.float32) * 4
    b = np.random.default_rng(5).standard_normal(n).astype(np.float32)
    o = torch.empty(n, device="cuda")
    kx.silu_mul_dev(dev(torch, a), dev(torch, b), o, n)
    ad = a.astype(np.float64)
    close(o.cpu().numpy(), ad * (1 / (1 + np.exp(-ad))) * b, rel=1e-6, abs_=1e-6)
    if L.ref() is not None:   # the reference's silu (f32_ops.c) then its multiply
        s = np.empty_like(a)
        L.ref().skainet_f32_unary(2, L.fp(a), L.fp(s), n)
        close(o.cpu().numpy(), s * b, rel=1e-6, abs_=1e-6)
    kx.add_dev(dev(torch, a), dev(torch, b), o, n)
    assert np.array_equal(o.cpu().numpy(), a + b)
    # arg-max: first maximum wins (TensorOps.argMax)
    lg = np.random.default_rng(6).standard_normal((4, 128256)).astype(np.float32)
    lg[1, 77] = lg[1, 90000] = 50.0
    lg[2, :] = -3.0
    lg[3, 128255] = 60.0
    idx = torch.empty(4, dtype=torch.int32, device="cuda")
    kx.argmax_rows_dev(dev(torch, lg), 4, 128256, idx)
    assert idx.cpu().tolist() == [int(lg[0].argmax()), 77, 0, 128255]
    # SPI kernels on host arrays
    norm, soft = kx.HipKernelProvider().norm_fp32(), kx.HipKernelProvider().softmax_fp32()
    ho = np.zeros((rows + 1, cols), np.float32)
    norm.rms_norm(x, cols, g, ho, cols, rows - 1, cols, 1e-5)     # offsets: skip the first row of both
    close(ho[1:rows], ref[1:rows], rel=1e-5)
    assert not ho[0].any() and not ho[rows].any()
    norm.layer_norm(x, 0, None, None, ho, 0, rows, cols, 1e-5)
    close(ho[:rows], (xd - mu) / np.sqrt(var + 1e-5), abs_=1e-4)
    soft.softmax_rows(x, 0, ho, 0, rows, cols, False)
    close(ho[:rows].sum(1), np.ones(rows), rel=1e-5)


@pytest.mark.parametrize("rows,cols", [(1, 8192), (3, 4099), (2, 100), (7, 6144), (1, 12288)])
def test_rms_norm_row_shapes(hip_backend, torch_cuda, rows, cols):
    """Register-cached rows (cols % 4 == 0 up to 8192) and the looping kernel (everything else) against the oracle."""
    torch, kx = torch_cuda, hip_backend
    x = (np.random.default_rng(cols).standard_normal((rows, cols)) * 2).astype(np.float32)
    g = np.random.default_rng(cols + 1).standard_normal(cols).astype(np.float32)
    out = torch.empty(rows, cols, device="cuda")
    kx.rms_norm_dev(dev(torch, x), dev(torch, g), out, rows, cols, 1e-6)
    ref = np.empty_like(x)
    L.oracle().orc_f32_rms_norm(L.fp(x), L.fp(g), L.fp(ref), rows, cols, 1e-6)
    close(out.cpu().numpy(), ref, rel=2e-5, abs_=1e-6)


@pytest.mark.parametrize("rows,cols", [(1, 16384), (64, 20000), (65, 20000), (2, 16383), (3, 128256)])
def test_argmax_split_and_single_kernels(hip_backend, torch_cuda, rows, cols):
    """Few long rows take the many-workgroups-per-row kernel (twice in a row: its counters must come back to zero),
    other shapes the one-workgroup-per-row kernel; ties keep the lowest index, also across slice borders."""
    torch, kx = torch_cuda, hip_backend
    lg = np.random.default_rng(rows * cols).standard_normal((rows, cols)).astype(np.float32)
    lg[0, cols - 1] = lg[0, cols // 2] = 40.0          # tie in two different slices
    if rows > 1:
        lg[1, :] = 1.5                                  # all equal: index 0
    idx = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    want = [int(r.argmax()) for r in lg]
    assert want[0] == cols // 2
    d = dev(torch, lg)
    for _ in range(2):
        idx.fill_(-1)
        kx.argmax_rows_dev(d, rows, cols, idx)
        assert idx.cpu().tolist() == want


def test_dense_matmuls(hip_backend, torch_cuda):
    prov = hip_backend.HipKernelProvider()
    # capability answers of KernelProvider.supports (KernelProvider.kt:161-190)
    for op in ("softmax", "layer_norm", "rms_norm", "sdpa"):
        assert prov.supports(op, ["Float32"]) and not prov.supports(op, ["Float16"])
    assert prov.supports("matmul_wt", ["Float32", "Float32"]) and not prov.supports("matmul_wt", ["Float32", "Q4_K"])
    assert not prov.supports("matmul", ["Float16", "Float32"]) and not prov.supports("matmul", ["Float32", "Q3_K"])
    assert not prov.supports("gather", ["Float32"]) and not prov.supports("matmul", ["Float32"])
    rng = np.random.default_rng(9)
    a = rng.standard_normal((70, 130)).astype(np.float32)
    b = rng.standard_normal((130, 90)).astype(np.float32)
    c = np.full((70, 100), 3.0, np.float32)
    # strided views: A rows 2.., 100 of 130 columns; C written into a wider matrix at an offset
    prov.matmul_fp32().matmul(a, 2 * 130 + 5, 130, b, 7, 90, c, 100 + 4, 100, 60, 80, 100)
    bb = np.lib.stride_tricks.as_strided(b.reshape(-1)[7:], (100, 80), (360, 4))
    want = a[2:62, 5:105].astype(np.float64) @ bb
    close(c[1:61, 4:84], want, rel=1e-5, abs_=1e-4)
    assert (c[0] == 3).all() and (c[1:61, :4] == 3).all() and (c[1:61, 84:] == 3).all() and (c[61:] == 3).all()
    ref = np.full((70, 100), 3.0, np.float32)
    L.oracle().orc_fp32_matmul(L.fp(a), 2 * 130 + 5, 130, L.fp(b), 7, 90, L.fp(ref), 104, 100, 60, 80, 100)
    close(c, ref, rel=1e-5, abs_=1e-4)
    z = np.full((4, 6), 9.0, np.float32)
    prov.matmul_fp32().matmul(a, 0, 130, b, 0, 90, z, 0, 6, 4, 6, 0)     # k == 0 zeroes C
    assert not z.any()
    w = rng.standard_normal((33, 130)).astype(np.float32)
    o = np.zeros((70, 33), np.float32)
    prov.matmul_fp32_wt().matmul_wt(a, 0, w, 0, o, 0, 70, 33, 130)
    close(o, a.astype(np.float64) @ w.T, rel=1e-5, abs_=1e-4)


@pytest.mark.parametrize("m,n,k,wt", [(512, 1024, 768, False), (200, 300, 260, False), (64, 32, 4, True), (130, 4096, 516, True),
                                      (1000, 132, 2048, False), (65, 257, 100, True)])
def test_dense_fp32_matmul_on_the_matrix_cores(hip_backend, torch_cuda, m, n, k, wt):
    """fp32 operands on the fp32 matrix instruction (exact products, fp32 accumulation in the instruction's order):
    resident operands through the device entries, ragged tiles in every direction, K from one instruction step to many
    slices, both layouts of B; against fp64 and against the tile kernel that takes the same call when the matrix-core
    one is switched off. Products whose strides or alignment the matrix-core kernel does not read stay on the tile
    kernel."""
    torch = torch_cuda
    rng = np.random.default_rng(m + n + k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((n, k) if wt else (k, n)).astype(np.float32)
    want = a.astype(np.float64) @ (b.astype(np.float64).T if wt else b.astype(np.float64))

    def run():
        out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
        if wt:
            hip_backend.fp32_matmul_wt_dev(dev(torch, a), 0, dev(torch, b), 0, out, 0, m, n, k)
        else:
            hip_backend.fp32_matmul_dev(dev(torch, a), 0, k, dev(torch, b), 0, n, out, 0, n, m, n, k)
        return out.cpu().numpy()

    got = run()
    assert hip_backend.last_kernel() == "sgemm_mfma_kernel"
    close(got, want, rel=1e-5, abs_=2e-6 * np.sqrt(k) * 16)
    try:
        hip_backend.set_tuning("dense_mfma", 0)
        tile = run()
        assert hip_backend.last_kernel() == "sgemm_kernel"
    finally:
        hip_backend.set_tuning("dense_mfma", 1)
    close(got, tile, rel=1e-5, abs_=2e-6 * np.sqrt(k) * 16)
    if not wt:
        # the same product out of a wider A at an offset of one float: not 16-byte aligned, the tile kernel's business
        wide = np.zeros((m, k + 4), np.float32)
        wide[:, 1:k + 1] = a
        out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
        hip_backend.fp32_matmul_dev(dev(torch, wide), 1, k + 4, dev(torch, b), 0, n, out, 0, n, m, n, k)
        assert hip_backend.last_kernel() == "sgemm_kernel"
        close(out.cpu().numpy(), want, rel=1e-5, abs_=2e-6 * np.sqrt(k) * 16)


@pytest.mark.parametrize("kind,codec", [("bf16", "BFloat16"), ("fp16", "Float16")])
def test_narrow_float_matmuls(hip_backend, torch_cuda, kind, codec):
    """Bf16MatmulKernel / Fp16MatmulKernel through the host entry: the oracle on the recorded inputs (with the formats'
    specials), then a ragged larger product with offsets, an odd byte offset and a padded byte row stride for B."""
    from test_oracle_golden import narrow_inputs, narrow_values
    prov = hip_backend.HipKernelProvider()
    kern = prov.matmul_bf16() if kind == "bf16" else prov.matmul_fp16()
    assert kern.codec == codec and prov.supports("matmul", ["Float32", codec])
    a, b, m, n, k = narrow_inputs(kind)
    c = np.full((m, n), np.nan, np.float32)
    kern.matmul(a, 0, k, b, 0, 2 * n, c, 0, n, m, n, k)
    want = L.narrow_matmul(kind, a, b, m, n, k)
    close(c, want.astype(np.float64), rel=1e-5, abs_=1e-6)
    recorded = np.load(os.path.join(HERE, "golden", "ref_vectors.npz"))[f"narrow/{kind}"]
    close(c, recorded.astype(np.float64), rel=1e-5, abs_=1e-6)
    # 70 x 83 x 150 out of wider buffers; B starts at an odd byte and its rows are 2 * 90 + 6 bytes apart
    rng = np.random.default_rng(12)
    m, n, k = 70, 83, 150
    a = rng.standard_normal((m + 2, k + 9)).astype(np.float32)
    bv = rng.standard_normal((k, n)).astype(np.float32)
    bits = (bv.view(np.uint32) >> 16).astype("<u2") if kind == "bf16" else bv.astype("<f2").view("<u2")
    stride = 2 * 90 + 6
    raw = np.full(3 + k * stride, 0xA5, np.uint8)
    rows = np.lib.stride_tricks.as_strided(raw[3:], (k, 2 * n), (stride, 1))
    rows[:] = np.ascontiguousarray(bits).view(np.uint8).reshape(k, 2 * n)
    c = np.full((m + 1, n + 5), 3.0, np.float32)
    kern.matmul(a, 2 * (k + 9) + 4, k + 9, raw, 3, stride, c, (n + 5) + 2, n + 5, m, n, k)
    want = a[2:, 4:4 + k].astype(np.float64) @ narrow_values(kind, np.ascontiguousarray(bits).view(np.uint8).reshape(-1), k, n).astype(np.float64)
    close(c[1:, 2:2 + n], want, rel=1e-5, abs_=1e-5)
    assert (c[0] == 3).all() and (c[:, :2] == 3).all() and (c[:, 2 + n:] == 3).all()
    ref = np.full_like(c, 3.0)
    getattr(L.oracle(), f"orc_{kind}_matmul")(L.fp(a), 2 * (k + 9) + 4, k + 9, L.u8(raw), 3, stride, L.fp(ref), (n + 5) + 2, n + 5, m, n, k)
    close(c, ref.astype(np.float64), rel=1e-5, abs_=1e-5)
    z = np.full((4, 6), 9.0, np.float32)
    kern.matmul(a, 0, k + 9, raw, 0, stride, z, 0, 6, 4, 6, 0)              # k == 0 zeroes C
    assert not z.any()
    with pytest.raises(ValueError):
        kern.matmul(a, 0, k + 9, raw, 0, stride, z, 0, 6, 4, 6, -1)


def test_thread_release_frees_and_regrows_scratch(hip_backend, torch_cuda):
    """A worker thread's scratch can be handed back (skainet_hip_thread_release); calls after it allocate afresh and
    give the same bits, and the memory the thread held is free again."""
    import threading
    from oracle import golden as G
    torch = torch_cuda
    provider = hip_backend.HipKernelProvider()
    n, nblocks = 96, 4
    k = nblocks * 256
    blocks = G.weight_blocks("Q4_K", n, nblocks, 0x5EED0700)
    x = G.floats(k, 0x5EED0701)
    want = L.gemv("Q4_K", x, G.row_major(blocks), n)
    b, h, hkv, skv, d = 2, 8, 2, 300, 64           # decode shape: split partials live in the thread's workspace
    q, kk, vv = sdpa_inputs(b, h, hkv, 1, skv, d, 31)
    results, errors = {}, []

    def worker():
        try:
            kernel = provider.matmul_q4k()
            att = provider.attention_fp32()
            for tag in ("before", "after"):
                y = np.zeros(n, np.float32)
                kernel.matmul_row_major(x, 0, G.row_major(blocks), 0, k, n, y, 0)
                o = np.zeros(b * h * d, np.float32)
                att.sdpa(q, kk, vv, o, b, h, hkv, 1, skv, d, 0.125, True, 0, 0)
                big = np.ones((4096, 4096), np.float32)              # 64 MiB staged on the device by the host-pointer entry
                provider.norm_fp32().rms_norm(big, 0, np.ones(4096, np.float32), np.empty_like(big), 0, 4096, 4096, 1e-5)
                results[tag] = (y, o)
                if tag == "before":
                    hip_backend.sync()
                    held = torch.cuda.mem_get_info()[0]
                    hip_backend.thread_release()
                    results["freed"] = torch.cuda.mem_get_info()[0] - held
            hip_backend.thread_release()
            hip_backend.thread_release()                              # idempotent
        except Exception as e:                                        # surfaced in the main thread below
            errors.append(e)

    t = threading.Thread(target=worker)
    t.start()
    t.join()
    assert not errors, errors
    assert normalized_err(results["before"][0], want) <= 1e-3
    assert np.array_equal(results["before"][0], results["after"][0])
    assert np.array_equal(results["before"][1], results["after"][1])
    assert results["freed"] >= 64 << 20, results["freed"]
